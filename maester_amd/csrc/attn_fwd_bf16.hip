// GQA flash-style forward for bf16 activations on gfx950 matrix cores.
//
// Stands in for the FlexAttention forward GemmaAttention.forward calls
// (maester/models/gemma/model.py:384-396; semantics torch/_higher_order_ops/flex_attention.py:159-267).
//
// One workgroup (4 waves) owns a 128-row q tile of one (batch row, q head); wave w owns rows
// 32w..32w+31 and keeps their Q fragments, the fp32 O^T accumulator and the online-softmax state in
// registers.  K/V are walked 64 rows at a time through LDS tiles, following the kv lists of the
// tile map (partial tiles first, then full tiles -- fully masked tiles are never touched); the
// global loads of step n+1 are in flight while step n is computed.
// Per step:  S^T = K Q^T (MFMA 32x32x16, K row fragments x Q registers), fp32 online softmax in
// the exp2 domain with the lane owning one q row (row max/sum = in-lane reduction + one 32-lane
// exchange), P^T cast to bf16 in place, O^T += V^T P^T (MFMA, V through transposed LDS reads).
// Inside partial tiles the 32-row kv blocks a wave cannot see under the causal/window bound are
// skipped, the rest is masked element-wise with the document/causal/window predicate.
#include "common.h"
#include "mfma.h"

constexpr int kPairMinD = 256;  // below that the one-head kernel fits two workgroups per compute unit, which beats sharing K/V fragments

namespace ma {

constexpr int kFwdThreads = 256;
constexpr int kFwdBN = 64;  // kv rows per step

constexpr int kPipe = 4;  // LDS fragment reads kept in flight ahead of the MFMAs

template <int D, bool HAS_DOC>
__device__ __forceinline__ void attn_fwd_bf16_item(KernArgs& a, const int wg_id) {
    using TL = Tile<D>;
    constexpr int KK = D / 16;  // contraction steps of S^T
    constexpr int DB = D / 32;  // 32-row blocks of O^T
    constexpr int BN = kFwdBN;
    extern __shared__ __align__(16) char smem_raw[];
    // double-buffered K and V tiles and kv document ids
    const lds_ptr lds0 = (lds_ptr)smem_raw;
    auto Kbuf = [&](int i) { return lds0 + i * 2 * TL::bytes(BN); };
    auto Vbuf = [&](int i) { return lds0 + i * 2 * TL::bytes(BN) + TL::bytes(BN); };
    auto Dbuf = [&](int i) { return (MA_LDS int64_t*)(lds0 + 4 * TL::bytes(BN)) + i * BN; };

    const int tid = fresh_tid(), lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keep it in a scalar register
    const int r = lane & 31, hh = lane >> 5;
    int i, h, b;
    if (!map_work(wg_id, a.B * a.T, a.T, a.Hkv, a.Hq / a.Hkv, a.map.q_tile_order, i, h, b)) return;
    const int hk = h / (a.Hq / a.Hkv);
    const int qw_lo = i * kTile + 32 * w, qw_hi = qw_lo + 31;
    const int q = qw_lo + r;
    const bool qvalid = q < a.S;
    const bool bounded = a.causal || a.window >= 0;  // kv <= q is part of the predicate

    const __bf16* qp = (const __bf16*)a.q.ptr + b * a.q.stride_b + h * a.q.stride_h;
    const char* kp = (const char*)((const __bf16*)a.k.ptr + b * a.k.stride_b + hk * a.k.stride_h);
    const char* vp = (const char*)((const __bf16*)a.v.ptr + b * a.v.stride_b + hk * a.v.stride_h);
    const uint32_t ksb = (uint32_t)(a.k.stride_s * 2), vsb = (uint32_t)(a.v.stride_s * 2);  // row strides in bytes
    const int64_t* drow = HAS_DOC ? a.doc + (size_t)b * a.S : nullptr;
    const int rbase = TL::row_base(lane), tbase = TL::tr_base(lane);

    // The Q tile comes in through LDS (coalesced 1 KB runs instead of 32 strided rows per load); it
    // borrows the second K/V buffer pair, which the first step does not use yet.  Its loads go out
    // first: they depend on nothing but the work item.
    {
        DirectStager<D, kTile, kFwdThreads / 64> sq;
        sq.init(w, lane);
        sq.issue(qp + (int64_t)i * kTile * a.q.stride_s, Kbuf(1), w, lane, min(kTile, a.S - i * kTile), a.q.stride_s);
    }

    // rows past the end of the sequence read the last valid row; their results are never stored
    const int qc = min(q, a.S - 1);
    const int64_t docq = HAS_DOC ? drow[qc] : 0;
    const bool windowed = a.window >= 0;
    const int wlim = windowed ? (int)min(a.window, (int64_t)0x3fffffff) : 0x7fffffff;

    f32x16 o[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[db][v] = 0.f;
    float m = -INFINITY, lsum = 0.f;
    const float sl2 = a.scale * kLog2e;

    // kv steps of the workgroup's tile row, and the limits inside which a 32-row kv block of a
    // partial tile can be visible to this wave
    const size_t mrow = (size_t)b * a.T + i;
    StepWalk<BN> st;
    {
        int lo, hi;
        visibility_limits(false, i * kTile, i * kTile + kTile - 1, BN, bounded, wlim, windowed, lo, hi);
        int n_partial, n_full;
        scalar_load2(a.map.kv_num_blocks + mrow, a.map.full_kv_num_blocks + mrow, n_partial, n_full);
        st.init(a.map.kv_indices + mrow * a.T, n_partial, a.map.full_kv_indices + mrow * a.T, n_full, 1, false, a.S, lo, hi);
    }
    int blk_lo, blk_hi;
    visibility_limits(false, qw_lo, qw_hi, 32, bounded, wlim, windowed, blk_lo, blk_hi);
    // document-id ranges: of the wave's own q rows now, of the two kv blocks of a step at each step
    const bool use_rng = HAS_DOC && a.map.block_doc_range != nullptr;
    const int64_t* rng_row = use_rng ? a.map.block_doc_range + (size_t)b * (2 * ((a.S + 63) / 64)) * 2 : nullptr;
    DocRange own;
    if (use_rng) {
        own.load(rng_row + (size_t)(min(qw_lo, a.S - 1) / MA_DOC_BLOCK) * 2);
        own.ready();
    }

    DirectStager<D, BN, kFwdThreads / 64> sk;  // the K and V tiles have the same shape: one set of slots
    sk.init(w, lane);
    int64_t kd_next = 0;
    const int my_runs = decltype(sk)::runs_of(w);
    bool have = st.first();
    int k0 = st.r0;
    bool partial = st.partial;
    if (have) {
        const int rows_valid = min(BN, a.S - k0);
        sk.issue((const __bf16*)(kp + (uint64_t)(uint32_t)k0 * ksb), Kbuf(0), w, lane, rows_valid, a.k.stride_s);
        sk.issue((const __bf16*)(vp + (uint64_t)(uint32_t)k0 * vsb), Vbuf(0), w, lane, rows_valid, a.v.stride_s);
        if (HAS_DOC && partial && tid < BN) kd_next = drow[min(k0 + tid, a.S - 1)];
    }
    bf16x8 qf[KK];
    {
        lds_ptr Qs = Kbuf(1);
        wait_vmem();
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) qf[kk] = TL::row_frag(Qs, rbase, 32 * w, kk);
        __syncthreads();  // all Q fragments are in registers before the buffers are reused
    }

    for (int n = 0; have; ++n) {
        const int cur = n & 1;
        lds_ptr Ks = Kbuf(cur), Vs = Vbuf(cur);
        MA_LDS int64_t* kdoc = Dbuf(cur);
        DocRange2 rng;
        if (use_rng && partial) rng.load(rng_row + (size_t)(k0 / MA_DOC_BLOCK) * 2);
        if (HAS_DOC && partial && tid < BN) kdoc[tid] = kd_next;
        wait_vmem();       // this wave's share of the current tiles has landed ...
        __syncthreads();   // ... and so has everyone's; all waves are also done with the other buffers

        const int ck0 = k0;
        const bool cpartial = partial;
        have = st.next();
        bool act[2];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) act[nb] = block_visible(ck0 + 32 * nb, a.S, cpartial, blk_lo, blk_hi);
        if (use_rng && cpartial) {  // no kv row of the block shares a document with the wave's q rows
            rng.ready();
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) act[nb] &= rng.meets(nb, own.lo(), own.hi());
        }
        const bool idle = !act[0] & !act[1];
        // The tile loads of the next step are spread over this step's two MFMA chains (K tile in the
        // first, V tile in the second), one run every few MFMAs: issued in one burst they fill the
        // memory pipeline and stall the wave with the matrix cores idle.  A ragged last tile, or a
        // step without chains, issues them at once.
        int pace = 0;
        const char *ksrc = kp, *vsrc = vp;
        if (have) {
            k0 = st.r0;
            partial = st.partial;
            ksrc = kp + (uint64_t)(uint32_t)k0 * ksb;
            vsrc = vp + (uint64_t)(uint32_t)k0 * vsb;
            if (HAS_DOC && partial && tid < BN) kd_next = drow[min(k0 + tid, a.S - 1)];
            pace = __builtin_amdgcn_readfirstlane(((k0 + BN <= a.S) & !idle) ? my_runs : 0);
            if (!pace) {
                const int rows_valid = min(BN, a.S - k0);
                sk.issue((const __bf16*)ksrc, Kbuf(cur ^ 1), w, lane, rows_valid, a.k.stride_s);
                sk.issue((const __bf16*)vsrc, Vbuf(cur ^ 1), w, lane, rows_valid, a.v.stride_s);
            }
        }
        if (idle) continue;
        const uint32_t kdst = lds_addr(Kbuf(cur ^ 1)), vdst = lds_addr(Vbuf(cur ^ 1));
        constexpr int kEvery = (2 * KK) / decltype(sk)::PER;  // both chains have 2*KK MFMAs
        static_assert(kEvery >= 1 && DB * 4 == 2 * KK, "pacing");
        auto pace_k = [&](auto idx) {
            constexpr int i = decltype(idx)::value;
            if constexpr (i % kEvery == kEvery - 1) sk.template issue_one<i / kEvery>((const __bf16*)ksrc, kdst, w, pace, ksb);
        };
        auto pace_v = [&](auto idx) {
            constexpr int i = decltype(idx)::value;
            if constexpr (i % kEvery == kEvery - 1) sk.template issue_one<i / kEvery>((const __bf16*)vsrc, vdst, w, pace, vsb);
        };

        // S^T blocks (kv x q).  Both 32-row blocks are always computed: a block the wave cannot see
        // is masked below, and keeping one straight-line path keeps every accumulator in place.
        f32x16 s[2];
        rowfrag_gemm<D, 2, kPipe>(lds_addr(Ks) + rbase, qf, s, pace_k);
        // mask (the scale into log2 units is folded into the exponent below)
        float mx = -INFINITY;
        if (cpartial) {
            // d = q - kv for element v is qrel - (32*nb + 8*(v/4) + v%4).  The causal, window and
            // end-of-sequence tests together are one range test dlo <= d <= dhi, done as a single
            // unsigned compare of (d - dlo) against (dhi - dlo).
            const int qrel = q - ck0 - 4 * hh;
            const int dlo = max(bounded ? 0 : -0x40000000, q - a.S + 1);   // kv <= q, kv < S
            const unsigned span = (unsigned)(wlim - dlo);                   // wlim >= dlo is not required:
            const bool some = wlim >= dlo;                                  // an empty range hides everything
            const unsigned t0 = (unsigned)(qrel - dlo);
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                // ids of the 16 kv rows of this block the lane owns: 4 groups of 4 consecutive rows
                i64x2 ids[4][2];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    ids[g][0] = ids[g][1] = i64x2{0, 0};
                    if (HAS_DOC) {
                        ids[g][0] = *(MA_LDS i64x2*)(kdoc + 32 * nb + 8 * g + 4 * hh);
                        ids[g][1] = *(MA_LDS i64x2*)(kdoc + 32 * nb + 8 * g + 4 * hh + 2);
                    }
                }
#pragma unroll
                for (int g = 0; g < 4; ++g) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int v = 4 * g + e;
                        bool ok = (t0 - (unsigned)(32 * nb + 8 * g + e) <= span) & some & act[nb];
                        if (HAS_DOC) ok = ok & (ids[g][e >> 1][e & 1] == docq);
                        const float x = ok ? s[nb][v] : -INFINITY;
                        s[nb][v] = x;
                        mx = fmaxf(mx, x);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);  // finish this block before starting the next
            }
        } else {
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
                for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[nb][v]);
            }
        }
        // the scores stay unscaled: the (positive) scale goes into the exponent's multiply-add below
        mx = fmaxf(mx, xor32(mx)) * sl2;
        // Lazy rescaling: the running reference m only moves when the row maximum has grown by more
        // than kSlack (in log2 units), so exp2(x - m) stays below 2^kSlack and the accumulator
        // rescale is a rare, wave-uniform branch instead of 128 multiplies per step.
        constexpr float kSlack = 8.0f;
        const bool grow = mx > m + kSlack;      // false while mx == -inf (nothing visible yet)
        if (__any(grow)) {
            const float mn = grow ? mx : m;
            const float alpha = m == -INFINITY ? 0.f : fast_exp2(m - mn);
            lsum *= alpha;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) o[db][v] *= alpha;
            m = mn;
        }
        const float mu = m == -INFINITY ? 0.f : m;
        float rs = 0.f;
        bf16x8 pf[2][2];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float p = fast_exp2(__builtin_fmaf(s[nb][v], sl2, -mu));
                rs += p;
                pf[nb][v >> 3][v & 7] = (__bf16)p;
            }
        }
        rs += xor32(rs);
        lsum += rs;

        // O^T += V^T P^T
        trfrag_gemm<D, 4, 6>(lds_addr(Vs) + tbase, &pf[0][0], o, pace_v);
    }

    // Epilogue: O^T (a lane owns one q row, 4 consecutive d per register group) goes through LDS so
    // that the global stores are whole 16-byte-per-lane row segments.
    __syncthreads();  // every wave is done with the K/V buffers
    mfma_fence();
    {
        constexpr int kPitchO = D * 2 + 16;
        lds_ptr Os = lds0 + w * 32 * kPitchO;
        const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                bf16x4 pk;
#pragma unroll
                for (int e = 0; e < 4; ++e) pk[e] = (__bf16)(o[db][4 * g + e] * inv);
                *(MA_LDS bf16x4*)(Os + r * kPitchO + (32 * db + 8 * g + 4 * hh) * 2) = pk;
            }
        }
        constexpr int CH = D / 8, RPI = 64 / CH;  // rows per store instruction
        const int rsub = lane / CH, c = lane % CH;
        __bf16* ob = (__bf16*)a.o.ptr + b * a.o.stride_b + h * a.o.stride_h;
#pragma unroll
        for (int it = 0; it < 32 / RPI; ++it) {
            const int row = it * RPI + rsub;
            const u32x4 val = *(MA_LDS u32x4*)(Os + row * kPitchO + c * 16);
            if (qw_lo + row < a.S) *(u32x4*)(ob + (int64_t)(qw_lo + row) * a.o.stride_s + c * 8) = val;
        }
        if (qvalid && hh == 0)
            a.lse[((size_t)b * a.Hq + h) * a.S + q] = lsum > 0.f ? (m + __log2f(lsum)) * kLn2 : -INFINITY;
    }
}

// One workgroup per work item, or -- with work queues in the tile map -- one per compute unit, pulling
// items until none is left (see WorkQueue).
template <int D, bool HAS_DOC>
__global__ __launch_bounds__(kFwdThreads) void attn_fwd_bf16_kernel(AttnArgs a) {
    extern __shared__ __align__(16) char smem_raw[];
    MA_LDS int* box = (MA_LDS int*)((lds_ptr)smem_raw + (4 * Tile<D>::bytes(kFwdBN) + 2 * kFwdBN * 8));
    WorkQueue wq;
    wq.init(a.map.work_counters, kQueueFwd, work_grid(a.B * a.T, a.Hkv, a.Hq / a.Hkv));
    for (int id = wq.next(box); id >= 0; id = wq.next(box)) {
        attn_fwd_bf16_item<D, HAS_DOC>(fresh_args(), id);
        __syncthreads();  // the item's LDS (and the box) are free again
    }
    wq.leave();
}

template <int D, bool HAS_DOC>
static int fwd_dd(const AttnArgs& a, hipStream_t st) {
    const size_t lds = (size_t)4 * Tile<D>::bytes(kFwdBN) + 2 * kFwdBN * 8 + 16;  // K/V ring, kv ids, work-queue box
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)attn_fwd_bf16_kernel<D, HAS_DOC>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return fail(MA_ERR_LAUNCH, "hipFuncSetAttribute(attn_fwd_bf16, %zu): %s", lds, hipGetErrorString(e));
    }
    static const int resident = resident_workgroups(attn_fwd_bf16_kernel<D, HAS_DOC>, kFwdThreads, lds);
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<D, HAS_DOC>), dim3(queue_grid(work_grid(a.B * a.T, a.Hkv, a.Hq / a.Hkv), a.map.work_counters, resident), 1, 1),
                       dim3(kFwdThreads), lds, st, a);
    return check_launch("attn_fwd_bf16_kernel");
}

template <int D>
static int fwd_d(const AttnArgs& a, hipStream_t st) {
    return a.doc ? fwd_dd<D, true>(a, st) : fwd_dd<D, false>(a, st);
}

int launch_attn_fwd_bf16(const AttnArgs& a, hipStream_t st) {
    // query heads that share a kv head are processed in pairs when they come in pairs
    if ((a.Hq / a.Hkv) % 2 == 0 && a.D >= kPairMinD) return launch_attn_fwd_pair_bf16(a, st);
    switch (a.D) {
        case 64: return fwd_d<64>(a, st);
        case 128: return fwd_d<128>(a, st);
        case 256: return fwd_d<256>(a, st);
    }
    return fail(MA_ERR_UNSUPPORTED, "attn_fwd bf16: head_dim %d not in {64,128,256}", a.D);
}

}  // namespace ma
