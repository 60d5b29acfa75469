// GQA flash-style backward for bf16 activations on gfx950 matrix cores.
//
// Stands in for the FlexAttention backward autograd runs for GemmaAttention
// (torch/_higher_order_ops/flex_attention.py:825-993):
//   delta = rowsum(O * dO);  P = exp(S - lse);  dV = P^T dO;  dS = P * (dO V^T - delta);
//   dQ = scale * dS K;  dK = scale * dS^T Q;  dK/dV summed over the query heads of a kv head.
// Two kernels (three when delta is asked for on its own), no atomics anywhere (results are
// run-to-run identical):
//   1. dQ: the forward's decomposition (128-row q tile per workgroup, 32 rows per wave, K/V
//      64 rows per step through LDS), recomputing S^T and dP^T; it also computes delta for its own
//      rows (it holds their dO fragments anyway) and writes it out for the second kernel;
//   2. dK/dV: one workgroup owns a 128-row kv tile of one (batch row, kv head), wave w its rows
//      32w..32w+31 (K, V fragments and the fp32 dK^T/dV^T accumulators in registers); it walks
//      the q-side lists of the tile map for each of the G query heads, 64 q rows per step
//      through LDS, recomputing S and dP;
//   (delta alone: one pass over O and dO.)
// All products are arranged so that P and dS stay in registers between the two MFMAs that
// produce and consume them (see mfma.h).
#include "common.h"
#include "mfma.h"

#ifndef MA_DKV_WAVES
#define MA_DKV_WAVES 1
#endif

namespace ma {

constexpr int kBwdThreads = 256;
constexpr int kStep = 64;   // rows staged per step
constexpr int kBPipe = 4;   // LDS fragment reads kept in flight ahead of the MFMAs

// O tile epilogue shared by the kernels: a wave holds a 32-row x D fp32 tile transposed in registers
// (lane (r, hh) owns row r and, per 32-column block, columns 8g + 4hh + e); it is scaled, cast to
// bf16, laid out row-major in the wave's LDS scratch and written out as 16-byte row segments.
template <int D>
__device__ __forceinline__ void store_tile_T(lds_ptr scratch, const f32x16* acc, float mul, __bf16* gbase, int64_t stride,
                                            int row0, int rows_end, int lane) {
    constexpr int DB = D / 32;
    constexpr int kPitchO = D * 2 + 16;
    const int r = lane & 31, hh = lane >> 5;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            bf16x4 pk;
#pragma unroll
            for (int e = 0; e < 4; ++e) pk[e] = (__bf16)(acc[db][4 * g + e] * mul);
            *(MA_LDS bf16x4*)(scratch + r * kPitchO + (32 * db + 8 * g + 4 * hh) * 2) = pk;
        }
    }
    constexpr int CH = D / 8, RPI = 64 / CH;
    const int rsub = lane / CH, c = lane % CH;
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) {
        const int row = it * RPI + rsub;
        const u32x4 val = *(MA_LDS u32x4*)(scratch + row * kPitchO + c * 16);
        if (row0 + row < rows_end) *(u32x4*)(gbase + (int64_t)(row0 + row) * stride + c * 8) = val;
    }
}

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
// WRITE_DS: every 32 x 32 block of every step the workgroup walks also leaves its dS^T in a.ds (zeros
// for a block the wave skips), for the dQ kernel that only multiplies it with K.
template <int D, bool HAS_DOC, bool WRITE_DS>
__device__ __forceinline__ void attn_bwd_dkv_bf16_item(KernArgs& a, const int wg_id) {
    using TL = Tile<D>;
    constexpr int KK = D / 16;
    constexpr int DB = D / 32;
    constexpr int BM = kStep;
    constexpr int NW = kBwdThreads / 64;
    extern __shared__ __align__(16) char smem_raw[];
    const lds_ptr lds0 = (lds_ptr)smem_raw;
    // ring of two (Q, dO) tile pairs, then per-row lse / delta / document id for the two steps
    auto Qbuf = [&](int i) { return lds0 + i * 2 * TL::bytes(BM); };
    auto Gbuf = [&](int i) { return lds0 + i * 2 * TL::bytes(BM) + TL::bytes(BM); };
    const lds_ptr aux = lds0 + 4 * TL::bytes(BM);
    auto Lbuf = [&](int i) { return (MA_LDS float*)(aux) + i * BM; };
    auto Ebuf = [&](int i) { return (MA_LDS float*)(aux + 2 * BM * 4) + i * BM; };
    auto Dbuf = [&](int i) { return (MA_LDS int64_t*)(aux + 4 * BM * 4) + i * BM; };

    const int tid = fresh_tid(), lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, hh = lane >> 5;
    int j, hk, b;
    if (!map_work(wg_id, a.B * a.T, a.T, a.Hkv, 1, a.map.kv_tile_order, j, hk, b)) return;
    const int rbase = TL::row_base(lane), tbase = TL::tr_base(lane);
    const int G = a.Hq / a.Hkv;
    const int kw_lo = j * kTile + 32 * w, kw_hi = kw_lo + 31;
    const int kv = kw_lo + r;
    const bool kvalid = kv < a.S;
    const bool bounded = a.causal || a.window >= 0;
    const float sl2 = a.scale * kLog2e;

    const __bf16* kp = (const __bf16*)a.k.ptr + b * a.k.stride_b + hk * a.k.stride_h;
    const __bf16* vp = (const __bf16*)a.v.ptr + b * a.v.stride_b + hk * a.v.stride_h;
    const int64_t* drow = HAS_DOC ? a.doc + (size_t)b * a.S : nullptr;
    const int kvc = min(kv, a.S - 1);
    const int64_t dock = HAS_DOC ? drow[kvc] : 0;
    const int wlim = a.window >= 0 ? (int)min(a.window, (int64_t)0x3fffffff) : 0x7fffffff;

    // K and V rows of the workgroup come in through LDS (coalesced) and stay in registers
    bf16x8 kf[KK], vf[KK];
    {
        DirectStager<D, kTile, NW> sk, sv;
        sk.init(w, lane);
        sv.init(w, lane);
        const int rows_valid = min(kTile, a.S - j * kTile);
        sk.issue(kp + (int64_t)j * kTile * a.k.stride_s, Qbuf(0), w, lane, rows_valid, a.k.stride_s);
        sv.issue(vp + (int64_t)j * kTile * a.v.stride_s, Qbuf(1), w, lane, rows_valid, a.v.stride_s);
        wait_vmem();
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            kf[kk] = TL::row_frag(Qbuf(0), rbase, 32 * w, kk);
            vf[kk] = TL::row_frag(Qbuf(1), rbase, 32 * w, kk);
        }
        __syncthreads();
    }

    f32x16 dkacc[DB], dvacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) dkacc[db][v] = dvacc[db][v] = 0.f;

    const size_t mrow = (size_t)b * a.T + j;
    // q steps of the kv tile, for each of the G query heads in turn, from the last q tile down (see
    // ListWalk); limits inside which a 32-row q block of a partial tile can be visible to this wave
    const bool windowed = a.window >= 0;
    int blk_lo, blk_hi;
    visibility_limits(true, kw_lo, kw_hi, 32, bounded, wlim, windowed, blk_lo, blk_hi);
    // document-id range of the wave's own kv rows (the step table tests the q blocks against it)
    const bool use_rng = HAS_DOC && a.map.block_doc_range != nullptr;
    const int64_t* rng_row = use_rng ? a.map.block_doc_range + (size_t)b * (2 * ((a.S + 63) / 64)) * 2 : nullptr;
    DocRange own;
    if (use_rng) {
        own.load(rng_row + (size_t)(min(kw_lo, a.S - 1) / MA_DOC_BLOCK) * 2);
        own.ready();
    }
    StepTable<BM, WRITE_DS> st;
    if (WRITE_DS) st.numbering(a.map.tile_slot, (int64_t)b * a.T * a.T + j, a.T);     // tile (i, j) of this batch row, i walked
    {
        int lo, hi;
        visibility_limits(true, j * kTile, j * kTile + kTile - 1, BM, bounded, wlim, windowed, lo, hi);
        int n_partial, n_full;
        scalar_load2(a.map.q_num_blocks + mrow, a.map.full_q_num_blocks + mrow, n_partial, n_full);
        st.init(a.map.q_indices + mrow * a.T, n_partial, a.map.full_q_indices + mrow * a.T, n_full, G, true, a.S, lo, hi,
                blk_lo, blk_hi, rng_row, use_rng ? own.lo() : 0, use_rng ? own.hi() : 0,
                (MA_LDS uint32_t*)(aux + 2 * BM * (4 + 4 + 8) + 16) + w * 128);
        st.prime();
    }

    DirectStager<D, BM, NW> sq;  // the Q and dO tiles have the same shape: one set of slots
    sq.init(w, lane);
    const uint32_t qsb = (uint32_t)(a.q.stride_s * 2), gsb = (uint32_t)(a.dout.stride_s * 2);  // row strides in bytes
    const char* qhead = (const char*)((const __bf16*)a.q.ptr + b * a.q.stride_b);
    const char* ghead = (const char*)((const __bf16*)a.dout.ptr + b * a.dout.stride_b);
    float lse_next = 0.f, dl_next = 0.f;
    int64_t qd_next = 0;
    // global sources of the step the iterator stands on
    const char *qsrc = nullptr, *gsrc = nullptr;
    auto locate = [&]() {
        const int h = hk * G + st.rep;
        qsrc = qhead + (uint64_t)(uint32_t)h * (uint32_t)(a.q.stride_h * 2) + (uint64_t)(uint32_t)st.r0 * qsb;
        gsrc = ghead + (uint64_t)(uint32_t)h * (uint32_t)(a.dout.stride_h * 2) + (uint64_t)(uint32_t)st.r0 * gsb;
    };
    auto issue_rows = [&]() {  // per-row lse / delta / document id of that step
        if (tid < BM) {
            const int h = hk * G + st.rep;
            const int qq = min(st.r0 + tid, a.S - 1);
            const size_t row = ((size_t)b * a.Hq + h) * a.S + qq;
            lse_next = a.lse[row];  // converted to log2 units when it is written to LDS
            dl_next = a.delta[row];
            if (HAS_DOC) qd_next = drow[qq];
        }
    };
    auto issue_q = [&](int buf) { sq.issue((const __bf16*)qsrc, Qbuf(buf), w, lane, min(BM, a.S - st.r0), a.q.stride_s); };
    auto issue_g = [&](int buf) { sq.issue((const __bf16*)gsrc, Gbuf(buf), w, lane, min(BM, a.S - st.r0), a.dout.stride_s); };
    const int my_runs = decltype(sq)::runs_of(w);
    bool have = st.next();
    int q0 = st.r0, rep = st.rep, tslot = st.tile_slot;
    bool partial = st.partial, act0 = st.act0, act1 = st.act1;
    if (have) {
        locate();
        issue_q(0);
        issue_g(0);
        issue_rows();
    }
    // Where the dS^T of a step goes: the slot of (head, visited tile) in a.ds and, inside it, the half of
    // the q tile the step covers -- a uniform address, formed on the scalar side; the lane adds the
    // byte offset of its kv row and of its 8 columns, the block and the column pair are immediates.
    auto ds_step = [&](int head, int q_first, int tile_slot) {
        const uint64_t slot = (uint64_t)(uint32_t)head * (uint64_t)a.ds_tiles + (uint32_t)tile_slot;
        return (char*)a.ds + slot * (kTile * kTile * 2) + (uint32_t)__builtin_amdgcn_readfirstlane((q_first & (kTile - 1)) * 2);
    };
    const uint32_t ds_lane = (uint32_t)((32 * w + r) * (kTile * 2) + 16 * hh);

    for (int n = 0; have; ++n) {
        const int cur = n & 1;
        const lds_ptr Qs = Qbuf(cur), Gs = Gbuf(cur);
        MA_LDS float* lse2s = Lbuf(cur);
        MA_LDS float* dls = Ebuf(cur);
        MA_LDS int64_t* qdoc = Dbuf(cur);
        if (tid < BM) {
            lse2s[tid] = lse_next * kLog2e;
            dls[tid] = dl_next;
            if (HAS_DOC) qdoc[tid] = qd_next;
        }
        wait_vmem();
        __syncthreads();

        const int cq0 = q0;
        const bool cpartial = partial;
        const bool skip[BM / 32] = {!act0, !act1};  // blocks in which this wave has nothing to do
        char* ds_out = WRITE_DS ? ds_step(hk * G + rep, cq0, tslot) : nullptr;
        have = st.next();
        // The tile loads of the next step are spread over this step's first MFMA chains, one run
        // every few MFMAs (Q tile in the first 32-row block, dO tile in the second): issued in one
        // burst they fill the memory pipeline and stall the wave with the matrix cores idle.  A
        // ragged last tile, or a block that is skipped, issues its tile at once.
        int pace = 0;
        if (have) {
            q0 = st.r0;
            rep = st.rep;
            tslot = st.tile_slot;
            partial = st.partial;
            act0 = st.act0;
            act1 = st.act1;
            locate();
            issue_rows();
            const bool spread = (q0 + BM <= a.S) & !skip[0] & !skip[1];
            pace = __builtin_amdgcn_readfirstlane(spread ? my_runs : 0);
            if (!pace) {
                issue_q(cur ^ 1);
                issue_g(cur ^ 1);
            }
        }
        const uint32_t qdst = lds_addr(Qbuf(cur ^ 1)), gdst = lds_addr(Gbuf(cur ^ 1));

#pragma unroll 1
        for (int mb = 0; mb < BM / 32; ++mb) {
            const int qb0 = cq0 + 32 * mb;
            if (mb ? skip[1] : skip[0]) {
                if (WRITE_DS) {
#pragma unroll
                    for (int pr = 0; pr < 2; ++pr) *(u32x4*)(ds_out + ds_lane + 64 * mb + 32 * pr) = u32x4{0, 0, 0, 0};
                }
                continue;
            }
            const __bf16* psrc = (const __bf16*)(mb ? gsrc : qsrc);
            const uint32_t pdst = mb ? gdst : qdst, psb = mb ? gsb : qsb;
            constexpr int kEvery = (2 * KK) / decltype(sq)::PER;
            static_assert(kEvery >= 1, "pacing");
            auto pace_hook = [&](auto idx) {
                constexpr int i = decltype(idx)::value;
                if constexpr (i % kEvery == kEvery - 1) sq.template issue_one<i / kEvery>(psrc, pdst, w, pace, psb);
            };

            // S = Q K^T and dP = dO V^T for 32 q rows x the wave's 32 kv rows (lane owns one kv row)
            f32x16 s, dp;
            const uint32_t roff = (uint32_t)(32 * mb * TL::kPitch);
            rowfrag_gemm2<D, kBPipe, false, false>(lds_addr(Qs) + rbase + roff, kf, s, lds_addr(Gs) + rbase + roff, vf, dp, pace_hook);

            bf16x8 pf[2], dsf[2];
            // d = q - kv for element v is drel + 8*(v/4) + v%4; range test as one unsigned compare
            const int drel = qb0 + 4 * hh - kv;
            const int dlo = bounded ? 0 : -0x40000000;
            const int dhi = min(wlim, a.S - 1 - kv);              // q - kv <= window, q < S
            const unsigned span = (unsigned)(dhi - dlo);
            const bool some = (dhi >= dlo) & kvalid;
            const unsigned t0 = (unsigned)(drel - dlo);
            // one straight-line body per kind of tile (masked / unmasked): a test inside the element
            // loop would turn into a branch per element
            auto elementwise = [&](auto masked_c) {
                constexpr bool MASKED = decltype(masked_c)::value;
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const int qoff = 32 * mb + 8 * g4 + 4 * hh;
                    const f32x4 l4 = *(MA_LDS f32x4*)(lse2s + qoff);
                    const f32x4 e4 = *(MA_LDS f32x4*)(dls + qoff);
                    i64x2 ida = {0, 0}, idb = {0, 0};
                    if (HAS_DOC && MASKED) {
                        ida = *(MA_LDS i64x2*)(qdoc + qoff);
                        idb = *(MA_LDS i64x2*)(qdoc + qoff + 2);
                    }
                    const int64_t ids[4] = {ida[0], ida[1], idb[0], idb[1]};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int v = 4 * g4 + e;
                        float p = fast_exp2(s[v] * sl2 - l4[e]);
                        if (MASKED) {
                            bool ok = (t0 + (unsigned)(8 * g4 + e) <= span) & some;
                            if (HAS_DOC) ok = ok & (ids[e] == dock);
                            p = ok ? p : 0.f;
                        }
                        const float ds = p * (dp[v] - e4[e]);
                        pf[v >> 3][v & 7] = (__bf16)p;
                        dsf[v >> 3][v & 7] = (__bf16)ds;
                    }
                }
            };
            if (cpartial) elementwise(std::true_type{});
            else elementwise(std::false_type{});
            if (WRITE_DS) {
                // A lane holds q columns 8*g4 + 4*hh .. +3 of its kv row; swapping the second half of the
                // hh = 0 lanes with the first half of the hh = 1 lanes gives every lane 8 consecutive
                // columns (16*pair + 8*hh .. +7): one 16-byte store per pair instead of two of 8 bytes, and
                // the two lanes of a row write 32 adjacent bytes.
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    const u32x4 f = __builtin_bit_cast(u32x4, dsf[pr]);   // dwords 0,1: g4 = 2*pr, dwords 2,3: g4 = 2*pr + 1
                    const auto s0 = __builtin_amdgcn_permlane32_swap(f[0], f[2], false, false);
                    const auto s1 = __builtin_amdgcn_permlane32_swap(f[1], f[3], false, false);
                    *(u32x4*)(ds_out + ds_lane + 64 * mb + 32 * pr) = u32x4{s0[0], s1[0], s0[1], s1[1]};
                }
            }
            // dV^T += dO^T P and dK^T += Q^T dS  (accumulators stay in AGPRs)
            // (one read pipeline for both products: it is filled once, and one fence serves both)
            trfrag_gemm_two<D, 2, kBPipe>(lds_addr(Gs) + tbase + roff, pf, dvacc, lds_addr(Qs) + tbase + roff, dsf, dkacc);
        }
    }

    __syncthreads();  // everyone is done with the tiles: reuse the ring as store scratch
    mfma_fence();
    {
        constexpr int kPitchO = D * 2 + 16;
        const lds_ptr scratch = lds0 + w * 32 * kPitchO;
        __bf16* okp = (__bf16*)a.dk.ptr + b * a.dk.stride_b + hk * a.dk.stride_h;
        __bf16* ovp = (__bf16*)a.dv.ptr + b * a.dv.stride_b + hk * a.dv.stride_h;
        store_tile_T<D>(scratch, dkacc, a.scale, okp, a.dk.stride_s, kw_lo, a.S, lane);
        store_tile_T<D>(scratch, dvacc, 1.0f, ovp, a.dv.stride_s, kw_lo, a.S, lane);
    }
}

// One workgroup per work item, or -- with work queues in the tile map -- one per compute unit, pulling
// items until none is left (see WorkQueue).
template <int D, bool HAS_DOC, bool WRITE_DS>
__global__ __launch_bounds__(kBwdThreads, D <= 128 ? MA_DKV_WAVES : 1) void attn_bwd_dkv_bf16_kernel(AttnArgs a) {
    extern __shared__ __align__(16) char smem_raw[];
    MA_LDS int* box = (MA_LDS int*)((lds_ptr)smem_raw + (4 * Tile<D>::bytes(kStep) + 2 * kStep * (4 + 4 + 8)));
    WorkQueue wq;
    wq.init(a.map.work_counters, kQueueDkv, work_grid(a.B * a.T, a.Hkv, 1));
    for (int id = wq.next(box); id >= 0; id = wq.next(box)) {
        attn_bwd_dkv_bf16_item<D, HAS_DOC, WRITE_DS>(fresh_args(), id);
        __syncthreads();  // the item's LDS (and the box) are free again
    }
    wq.leave();
}

// ------------------------------------------------------------------------------------------------
// dQ
// ------------------------------------------------------------------------------------------------
template <int D, bool HAS_DOC>
__device__ __forceinline__ void attn_bwd_dq_bf16_item(KernArgs& a, const int wg_id) {
    using TL = Tile<D>;
    constexpr int KK = D / 16;
    constexpr int DB = D / 32;
    constexpr int BN = kStep;
    constexpr int NW = kBwdThreads / 64;
    extern __shared__ __align__(16) char smem_raw[];
    const lds_ptr lds0 = (lds_ptr)smem_raw;
    auto Kbuf = [&](int i) { return lds0 + i * 2 * TL::bytes(BN); };
    auto Vbuf = [&](int i) { return lds0 + i * 2 * TL::bytes(BN) + TL::bytes(BN); };
    auto Dbuf = [&](int i) { return (MA_LDS int64_t*)(lds0 + 4 * TL::bytes(BN)) + i * BN; };

    const int tid = fresh_tid(), lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, hh = lane >> 5;
    int i, h, b;
    if (!map_work(wg_id, a.B * a.T, a.T, a.Hkv, a.Hq / a.Hkv, a.map.q_tile_order, i, h, b)) return;
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
    const int64_t* drow = HAS_DOC ? a.doc + (size_t)b * a.S : nullptr;
    const int qc = min(q, a.S - 1);
    const int64_t docq = HAS_DOC ? drow[qc] : 0;
    const int wlim = a.window >= 0 ? (int)min(a.window, (int64_t)0x3fffffff) : 0x7fffffff;
    const size_t rowi = ((size_t)b * a.Hq + h) * a.S + qc;
    const float lse2 = a.lse[rowi] * kLog2e;
    // delta = rowsum(O * dO) of the wave's rows: computed here when the caller asked for that stage
    // together with this one (the dO rows are on hand anyway), read back otherwise
    const bool own_delta = (a.stages & MA_BWD_DELTA) != 0;
    float delta = own_delta ? 0.f : a.delta[rowi];

    // The walk over the kv tiles is set up first: its index loads are then ahead of the bulk loads
    // below in the memory pipeline, and the first K/V tiles can be requested as soon as they return.
    const size_t mrow = (size_t)b * a.T + i;
    const bool windowed = a.window >= 0;
    int blk_lo, blk_hi;
    visibility_limits(false, qw_lo, qw_hi, 32, bounded, wlim, windowed, blk_lo, blk_hi);
    // document-id range of the wave's own q rows (the step table tests the kv blocks against it)
    const bool use_rng = HAS_DOC && a.map.block_doc_range != nullptr;
    const int64_t* rng_row = use_rng ? a.map.block_doc_range + (size_t)b * (2 * ((a.S + 63) / 64)) * 2 : nullptr;
    DocRange own;
    if (use_rng) {  // (load and wait stay adjacent: the registers of a scalar load in flight must not be touched)
        own.load(rng_row + (size_t)(min(qw_lo, a.S - 1) / MA_DOC_BLOCK) * 2);
        own.ready();
    }
    StepTable<BN> st;
    {
        int lo, hi;
        visibility_limits(false, i * kTile, i * kTile + kTile - 1, BN, bounded, wlim, windowed, lo, hi);
        int n_partial, n_full;
        scalar_load2(a.map.kv_num_blocks + mrow, a.map.full_kv_num_blocks + mrow, n_partial, n_full);
        st.init(a.map.kv_indices + mrow * a.T, n_partial, a.map.full_kv_indices + mrow * a.T, n_full, 1, false, a.S, lo, hi,
                blk_lo, blk_hi, rng_row, use_rng ? own.lo() : 0, use_rng ? own.hi() : 0,
                (MA_LDS uint32_t*)(lds0 + 4 * TL::bytes(BN) + 2 * BN * 8 + 16) + w * 64);
        st.prime();
    }

    // Q and dO rows of the wave go straight from global memory into MFMA operand fragments: lane
    // (r, hh) holds elements 16*kk + 8*hh .. +7 of row qw_lo + r, one 16-byte load each (the two
    // halves of a wave read adjacent 16 bytes, every 128-byte line is used in full by four loads).
    // Nothing passes through LDS, so the index lists and the first K/V tiles are fetched at the
    // same time instead of after a barrier.
    bf16x8 qf[KK], gf[KK];
    u32x4 of[KK];
    {
        const __bf16* qrow = qp + (int64_t)qc * a.q.stride_s + 8 * hh;
        const __bf16* grow = gp + (int64_t)qc * a.dout.stride_s + 8 * hh;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) qf[kk] = *(const bf16x8*)(qrow + 16 * kk);
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) gf[kk] = *(const bf16x8*)(grow + 16 * kk);
        if (own_delta) {
            const __bf16* orow = (const __bf16*)a.o.ptr + b * a.o.stride_b + h * a.o.stride_h + (int64_t)qc * a.o.stride_s + 8 * hh;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) of[kk] = *(const u32x4*)(orow + 16 * kk);
        }
    }

    f32x16 acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[db][v] = 0.f;

    DirectStager<D, BN, NW> sk;  // the K and V tiles have the same shape: one set of slots
    sk.init(w, lane);
    const uint32_t ksb = (uint32_t)(a.k.stride_s * 2), vsb = (uint32_t)(a.v.stride_s * 2);  // row strides in bytes
    int64_t kd_next = 0;
    // the step the iterator stands on
    auto issue_k = [&](int buf) {
        sk.issue((const __bf16*)((const char*)kp + (uint64_t)(uint32_t)st.r0 * ksb), Kbuf(buf), w, lane, min(BN, a.S - st.r0), a.k.stride_s);
    };
    auto issue_v = [&](int buf) {
        sk.issue((const __bf16*)((const char*)vp + (uint64_t)(uint32_t)st.r0 * vsb), Vbuf(buf), w, lane, min(BN, a.S - st.r0), a.v.stride_s);
    };
    auto issue_ids = [&]() {
        if (HAS_DOC && st.partial && tid < BN) kd_next = drow[min(st.r0 + tid, a.S - 1)];
    };
    const int my_runs = decltype(sk)::runs_of(w);
    bool have = st.next();
    int k0 = st.r0;
    bool partial = st.partial, act0 = st.act0, act1 = st.act1;
    if (have) {
        issue_k(0);
        issue_v(0);
        issue_ids();
    }

    if (own_delta) {
        // lane (r, hh) sums its half of row r's products; the other half is in lane (r, 1 - hh)
        float sum = 0.f;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const u32x4 g = __builtin_bit_cast(u32x4, gf[kk]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {  // bf16 -> fp32 is a 16-bit shift
                sum += __builtin_bit_cast(float, of[kk][e] << 16) * __builtin_bit_cast(float, g[e] << 16);
                sum += __builtin_bit_cast(float, of[kk][e] & 0xffff0000u) * __builtin_bit_cast(float, g[e] & 0xffff0000u);
            }
        }
        delta = sum + xor32(sum);
        if (qvalid && hh == 0) a.delta[rowi] = delta;
    }
    // From here on the fragments are MFMA operands only: move them to AGPRs once, now.  (Left to
    // the register allocator, fragments that were also read by the vector ALU stay in VGPRs and
    // get copied to AGPRs right in front of every MFMA that uses them.)
    static_for<0, KK>([&](auto kk) { park_in_agprs(qf[decltype(kk)::value], gf[decltype(kk)::value]); });

    for (int n = 0; have; ++n) {
        const int cur = n & 1;
        const lds_ptr Ks = Kbuf(cur), Vs = Vbuf(cur);
        MA_LDS int64_t* kdoc = Dbuf(cur);
        if (HAS_DOC && partial && tid < BN) kdoc[tid] = kd_next;
        wait_vmem();
        __syncthreads();

        const int ck0 = k0;
        const bool cpartial = partial;
        const bool skip[BN / 32] = {!act0, !act1};  // blocks in which this wave has nothing to do
        have = st.next();
        // The tile loads of the next step are spread over this step's first MFMA chains (K tile in
        // the first 32-row block, V tile in the second), see the dK/dV kernel.
        int pace = 0;
        const __bf16 *ksrc = kp, *vsrc = vp;
        if (have) {
            k0 = st.r0;
            partial = st.partial;
            act0 = st.act0;
            act1 = st.act1;
            ksrc = (const __bf16*)((const char*)kp + (uint64_t)(uint32_t)k0 * ksb);
            vsrc = (const __bf16*)((const char*)vp + (uint64_t)(uint32_t)k0 * vsb);
            issue_ids();
            const bool spread = (k0 + BN <= a.S) & !skip[0] & !skip[1];
            pace = __builtin_amdgcn_readfirstlane(spread ? my_runs : 0);
            if (!pace) {
                issue_k(cur ^ 1);
                issue_v(cur ^ 1);
            }
        }
        const uint32_t kdst = lds_addr(Kbuf(cur ^ 1)), vdst = lds_addr(Vbuf(cur ^ 1));

#pragma unroll 1
        for (int nb = 0; nb < BN / 32; ++nb) {
            const int kb0 = ck0 + 32 * nb;
            if (nb ? skip[1] : skip[0]) continue;
            const __bf16* psrc = nb ? vsrc : ksrc;
            const uint32_t pdst = nb ? vdst : kdst, psb = nb ? vsb : ksb;
            constexpr int kEvery = (2 * KK) / decltype(sk)::PER;
            static_assert(kEvery >= 1, "pacing");
            // S^T = K Q^T, then dP^T = V dO^T, for 32 kv rows x the wave's 32 q rows (lane owns one q
            // row).  The two products run one after the other so that the exponentials of S^T (a
            // quarter-rate instruction each) are taken in the shadow of the dP^T MFMAs: one value
            // per MFMA, from the second MFMA after S^T is complete; what does not fit follows the chain.
            f32x16 s, dp;
            constexpr int kFirstExp = KK + 2, kHooked = (2 * KK - kFirstExp) < 16 ? (2 * KK - kFirstExp) : 16;
            auto chain_hook = [&](auto idx) {
                constexpr int i = decltype(idx)::value;
                if constexpr (i % kEvery == kEvery - 1) sk.template issue_one<i / kEvery>(psrc, pdst, w, pace, psb);
                if constexpr (i >= kFirstExp && i - kFirstExp < 16) s[i - kFirstExp] = fast_exp2(s[i - kFirstExp] * sl2 - lse2);
            };
            const uint32_t roff = (uint32_t)(32 * nb * TL::kPitch);
            rowfrag_gemm2<D, kBPipe, false, true, decltype(chain_hook)&, true>(lds_addr(Ks) + rbase + roff, qf, s, lds_addr(Vs) + rbase + roff, gf, dp,
                                                                                 chain_hook);
#pragma unroll
            for (int v = kHooked; v < 16; ++v) s[v] = fast_exp2(s[v] * sl2 - lse2);

            bf16x8 dsf[2];
            const int qrel = q - kb0 - 4 * hh;                     // d = q - kv = qrel - (8*(v/4) + v%4)
            const int dlo = max(bounded ? 0 : -0x40000000, q - a.S + 1);
            const unsigned span = (unsigned)(wlim - dlo);
            const bool some = (wlim >= dlo) & qvalid;
            const unsigned t0 = (unsigned)(qrel - dlo);
            auto elementwise = [&](auto masked_c) {  // one straight-line body per kind of tile
                constexpr bool MASKED = decltype(masked_c)::value;
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    i64x2 ida = {0, 0}, idb = {0, 0};
                    if (HAS_DOC && MASKED) {
                        ida = *(MA_LDS i64x2*)(kdoc + 32 * nb + 8 * g4 + 4 * hh);
                        idb = *(MA_LDS i64x2*)(kdoc + 32 * nb + 8 * g4 + 4 * hh + 2);
                    }
                    const int64_t ids[4] = {ida[0], ida[1], idb[0], idb[1]};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int v = 4 * g4 + e;
                        float p = s[v];  // exp2(S^T * scale - lse) by now
                        if (MASKED) {
                            bool ok = (t0 - (unsigned)(8 * g4 + e) <= span) & some;
                            if (HAS_DOC) ok = ok & (ids[e] == docq);
                            p = ok ? p : 0.f;
                        }
                        dsf[v >> 3][v & 7] = (__bf16)(p * (dp[v] - delta));
                    }
                }
            };
            if (cpartial) elementwise(std::true_type{});
            else elementwise(std::false_type{});
            // dQ^T += K^T dS^T  (accumulator stays in AGPRs)
            trfrag_gemm<D, 2, kBPipe, true>(lds_addr(Ks) + tbase + roff, dsf, acc);
        }
    }

    __syncthreads();
    mfma_fence();
    {
        constexpr int kPitchO = D * 2 + 16;
        __bf16* ob = (__bf16*)a.dq.ptr + b * a.dq.stride_b + h * a.dq.stride_h;
        store_tile_T<D>(lds0 + w * 32 * kPitchO, acc, a.scale, ob, a.dq.stride_s, qw_lo, a.S, lane);
    }
}

// One workgroup per work item.  (This kernel has many short items and no registers to spare: the
// work queues that the forward and dK/dV kernels pull from cost it more than they gain.)
template <int D, bool HAS_DOC>
__global__ __launch_bounds__(kBwdThreads, D <= 128 ? 2 : 1) void attn_bwd_dq_bf16_kernel(AttnArgs a) {
    attn_bwd_dq_bf16_item<D, HAS_DOC>(fresh_args(), (int)blockIdx.x);
}

// ------------------------------------------------------------------------------------------------
// dQ from the dS^T that the dK/dV kernel left in a.ds
// ------------------------------------------------------------------------------------------------
#ifndef MA_DQ_PAIR_MIN_D
#define MA_DQ_PAIR_MIN_D 64   // head dims from which an even GQA group goes through the two-head kernel
#endif
// dQ^T += K^T dS^T and nothing else: no Q / dO / O fragments, no scores, no exponentials.  Per step
// of 64 kv rows the workgroup stages the K tile and the [64 kv][128 q] slab of dS^T of its q tile;
// both MFMA operands come from LDS through transposed reads of the same kv rows, so their
// contraction orders agree by construction.  Every block this kernel reads has been written: it
// walks the same tile lists as the dK/dV kernel, that kernel writes all blocks of every step it
// walks, and a block that can hold a visible pair lies inside a step with a visible pair.
template <int D, bool HAS_DOC>
__device__ __forceinline__ void attn_bwd_dq_ds_bf16_item(KernArgs& a, const int wg_id) {
    using TL = Tile<D>;
    using TS = Tile<kTile>;
    constexpr int DB = D / 32;
    constexpr int BN = kStep;
    constexpr int NW = kBwdThreads / 64;
    extern __shared__ __align__(16) char smem_raw[];
    const lds_ptr lds0 = (lds_ptr)smem_raw;
    auto Kbuf = [&](int i) { return lds0 + i * TL::bytes(BN); };
    auto Sbuf = [&](int i) { return lds0 + 2 * TL::bytes(BN) + i * TS::bytes(BN); };

    const int tid = fresh_tid(), lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    int i, h, b;
    if (!map_work(wg_id, a.B * a.T, a.T, a.Hkv, a.Hq / a.Hkv, a.map.q_tile_order, i, h, b)) return;
    const int tbase = TL::tr_base(lane), sbase = TS::tr_base(lane);
    const int hk = h / (a.Hq / a.Hkv);
    const int qw_lo = i * kTile + 32 * w, qw_hi = qw_lo + 31;
    const bool bounded = a.causal || a.window >= 0;
    const __bf16* kp = (const __bf16*)a.k.ptr + b * a.k.stride_b + hk * a.k.stride_h;
    const __bf16* sp = (const __bf16*)a.ds + (size_t)h * (size_t)a.ds_tiles * (kTile * kTile);   // slot 0 of this head
    const int wlim = a.window >= 0 ? (int)min(a.window, (int64_t)0x3fffffff) : 0x7fffffff;

    const size_t mrow = (size_t)b * a.T + i;
    const bool windowed = a.window >= 0;
    int blk_lo, blk_hi;
    visibility_limits(false, qw_lo, qw_hi, 32, bounded, wlim, windowed, blk_lo, blk_hi);
    const bool use_rng = HAS_DOC && a.map.block_doc_range != nullptr;
    const int64_t* rng_row = use_rng ? a.map.block_doc_range + (size_t)b * (2 * ((a.S + 63) / 64)) * 2 : nullptr;
    DocRange own;
    if (use_rng) {  // (load and wait stay adjacent: the registers of a scalar load in flight must not be touched)
        own.load(rng_row + (size_t)(min(qw_lo, a.S - 1) / MA_DOC_BLOCK) * 2);
        own.ready();
    }
    StepTable<BN, true> st;
    st.numbering(a.map.tile_slot, ((int64_t)b * a.T + i) * a.T, 1);     // tile (i, j) of this batch row, j walked
    {
        int lo, hi;
        visibility_limits(false, i * kTile, i * kTile + kTile - 1, BN, bounded, wlim, windowed, lo, hi);
        int n_partial, n_full;
        scalar_load2(a.map.kv_num_blocks + mrow, a.map.full_kv_num_blocks + mrow, n_partial, n_full);
        st.init(a.map.kv_indices + mrow * a.T, n_partial, a.map.full_kv_indices + mrow * a.T, n_full, 1, false, a.S, lo, hi,
                blk_lo, blk_hi, rng_row, use_rng ? own.lo() : 0, use_rng ? own.hi() : 0,
                (MA_LDS uint32_t*)(lds0 + 2 * TL::bytes(BN) + 2 * TS::bytes(BN) + 16) + w * 128);
        st.prime();
    }

    f32x16 acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[db][v] = 0.f;

    DirectStager<D, BN, NW> sk;
    DirectStager<kTile, BN, NW> ss;
    sk.init(w, lane);
    ss.init(w, lane);
    const uint32_t ksb = (uint32_t)(a.k.stride_s * 2);
    auto issue = [&](int buf) {  // K rows r0 .. r0+63 and the matching 64 rows of dS^T (row r0 of the tile list = kv row)
        sk.issue((const __bf16*)((const char*)kp + (uint64_t)(uint32_t)st.r0 * ksb), Kbuf(buf), w, lane, min(BN, a.S - st.r0), a.k.stride_s);
        ss.issue(sp + (size_t)(uint32_t)st.tile_slot * (kTile * kTile) + (size_t)(st.r0 & (kTile - 1)) * kTile, Sbuf(buf), w, lane, BN, kTile);   // the step's 64 kv rows inside its tile's slot
    };
    bool have = st.next();
    bool act0 = st.act0, act1 = st.act1;
    if (have) issue(0);

    for (int n = 0; have; ++n) {
        const int cur = n & 1;
        const lds_ptr Ks = Kbuf(cur), Ss = Sbuf(cur);
        wait_vmem();
        __syncthreads();
        const bool skip[BN / 32] = {!act0, !act1};
        have = st.next();
        if (have) {
            act0 = st.act0;
            act1 = st.act1;
            issue(cur ^ 1);
        }
#pragma unroll 1
        for (int nb = 0; nb < BN / 32; ++nb) {
            if (nb ? skip[1] : skip[0]) continue;
            bf16x8 dsf[2];
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) dsf[jj] = TS::tr_frag(Ss, sbase, 32 * nb + 16 * jj, 32 * w);
            trfrag_gemm<D, 2, kBPipe, true>(lds_addr(Ks) + tbase + (uint32_t)(32 * nb * TL::kPitch), dsf, acc);
        }
    }

    __syncthreads();
    mfma_fence();
    {
        constexpr int kPitchO = D * 2 + 16;
        __bf16* ob = (__bf16*)a.dq.ptr + b * a.dq.stride_b + h * a.dq.stride_h;
        store_tile_T<D>(lds0 + w * 32 * kPitchO, acc, a.scale, ob, a.dq.stride_s, qw_lo, a.S, lane);
    }
}

template <int D, bool HAS_DOC>
__global__ __launch_bounds__(kBwdThreads, D <= 128 ? 2 : 1) void attn_bwd_dq_ds_bf16_kernel(AttnArgs a) {
    attn_bwd_dq_ds_bf16_item<D, HAS_DOC>(fresh_args(), (int)blockIdx.x);
}

// Two query heads of one kv head per workgroup: the K tile is staged once and every transposed K
// fragment read from LDS feeds two MFMAs (one per head's dS^T), which halves the kernel's K traffic
// and LDS reads per FLOP.  The tile loads of the next step are spread over this step's chains: the K
// tile over the first 32-row block, the two dS^T slabs over the second.
template <int D, bool HAS_DOC>
__device__ __forceinline__ void attn_bwd_dq_ds_pair_bf16_item(KernArgs& a, const int wg_id) {
    using TL = Tile<D>;
    using TS = Tile<kTile>;
    constexpr int DB = D / 32;
    constexpr int BN = kStep;
    constexpr int NW = kBwdThreads / 64;
    constexpr int kStage = TL::bytes(BN) + 2 * TS::bytes(BN);      // K tile, dS^T of head 0, dS^T of head 1
    extern __shared__ __align__(16) char smem_raw[];
    const lds_ptr lds0 = (lds_ptr)smem_raw;
    auto Kbuf = [&](int i) { return lds0 + i * kStage; };
    auto Sbuf = [&](int i, int head) { return lds0 + i * kStage + TL::bytes(BN) + head * TS::bytes(BN); };

    const int tid = fresh_tid(), lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int G = a.Hq / a.Hkv, GP = G / 2;
    int i, hp, b;
    if (!map_work(wg_id, a.B * a.T, a.T, a.Hkv, GP, a.map.q_tile_order, i, hp, b)) return;
    const int hk = hp / GP;
    const int h0 = hk * G + 2 * (hp % GP);  // the pair is (h0, h0 + 1)
    const int tbase = TL::tr_base(lane), sbase = TS::tr_base(lane);
    const int qw_lo = i * kTile + 32 * w, qw_hi = qw_lo + 31;
    const bool bounded = a.causal || a.window >= 0;
    const __bf16* kp = (const __bf16*)a.k.ptr + b * a.k.stride_b + hk * a.k.stride_h;
    const size_t head_slots = (size_t)a.ds_tiles * (kTile * kTile);
    const __bf16* sp0 = (const __bf16*)a.ds + (size_t)h0 * head_slots;   // slot 0 of the two heads
    const __bf16* sp1 = sp0 + head_slots;
    const int wlim = a.window >= 0 ? (int)min(a.window, (int64_t)0x3fffffff) : 0x7fffffff;

    const size_t mrow = (size_t)b * a.T + i;
    const bool windowed = a.window >= 0;
    int blk_lo, blk_hi;
    visibility_limits(false, qw_lo, qw_hi, 32, bounded, wlim, windowed, blk_lo, blk_hi);
    const bool use_rng = HAS_DOC && a.map.block_doc_range != nullptr;
    const int64_t* rng_row = use_rng ? a.map.block_doc_range + (size_t)b * (2 * ((a.S + 63) / 64)) * 2 : nullptr;
    DocRange own;
    if (use_rng) {  // (load and wait stay adjacent: the registers of a scalar load in flight must not be touched)
        own.load(rng_row + (size_t)(min(qw_lo, a.S - 1) / MA_DOC_BLOCK) * 2);
        own.ready();
    }
    StepTable<BN, true> st;
    st.numbering(a.map.tile_slot, ((int64_t)b * a.T + i) * a.T, 1);     // tile (i, j) of this batch row, j walked
    {
        int lo, hi;
        visibility_limits(false, i * kTile, i * kTile + kTile - 1, BN, bounded, wlim, windowed, lo, hi);
        int n_partial, n_full;
        scalar_load2(a.map.kv_num_blocks + mrow, a.map.full_kv_num_blocks + mrow, n_partial, n_full);
        st.init(a.map.kv_indices + mrow * a.T, n_partial, a.map.full_kv_indices + mrow * a.T, n_full, 1, false, a.S, lo, hi,
                blk_lo, blk_hi, rng_row, use_rng ? own.lo() : 0, use_rng ? own.hi() : 0,
                (MA_LDS uint32_t*)(lds0 + 2 * kStage + 16) + w * 128);
        st.prime();
    }

    f32x16 acc0[DB], acc1[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc0[db][v] = acc1[db][v] = 0.f;

    DirectStager<D, BN, NW> sk;
    DirectStager<kTile, BN, NW> ss;
    sk.init(w, lane);
    ss.init(w, lane);
    const uint32_t ksb = (uint32_t)(a.k.stride_s * 2);
    auto issue = [&](int buf) {
        sk.issue((const __bf16*)((const char*)kp + (uint64_t)(uint32_t)st.r0 * ksb), Kbuf(buf), w, lane, min(BN, a.S - st.r0), a.k.stride_s);
        const size_t at = (size_t)(uint32_t)st.tile_slot * (kTile * kTile) + (size_t)(st.r0 & (kTile - 1)) * kTile;
        ss.issue(sp0 + at, Sbuf(buf, 0), w, lane, BN, kTile);
        ss.issue(sp1 + at, Sbuf(buf, 1), w, lane, BN, kTile);
    };
    const int k_runs = decltype(sk)::runs_of(w), s_runs = decltype(ss)::runs_of(w);
    bool have = st.next();
    bool act0 = st.act0, act1 = st.act1;
    if (have) issue(0);

    for (int n = 0; have; ++n) {
        const int cur = n & 1;
        wait_vmem();
        __syncthreads();
        const bool skip0 = !act0, skip1 = !act1;
        have = st.next();
        int pace = 0;
        const __bf16 *ksrc = kp, *s0src = sp0, *s1src = sp1;
        if (have) {
            act0 = st.act0;
            act1 = st.act1;
            ksrc = (const __bf16*)((const char*)kp + (uint64_t)(uint32_t)st.r0 * ksb);
            const size_t at = (size_t)(uint32_t)st.tile_slot * (kTile * kTile) + (size_t)(st.r0 & (kTile - 1)) * kTile;
            s0src = sp0 + at;
            s1src = sp1 + at;
            // (smaller head dims have too few MFMAs per block to hide the runs behind: all at once)
            constexpr bool kPaced = decltype(sk)::PER <= (2 * 2 * DB) / 3 && 2 * decltype(ss)::PER <= (2 * 2 * DB) / 3;
            const bool spread = kPaced & (st.r0 + BN <= a.S) & !skip0 & !skip1;
            pace = __builtin_amdgcn_readfirstlane(spread ? 1 : 0);
            if (!pace) issue(cur ^ 1);
        }
        const uint32_t kdst = lds_addr(Kbuf(cur ^ 1)), s0dst = lds_addr(Sbuf(cur ^ 1, 0)), s1dst = lds_addr(Sbuf(cur ^ 1, 1));
        const int k_lim = pace ? k_runs : 0, s_lim = pace ? s_runs : 0;
        constexpr int kEvery = 3;                                   // one run every third MFMA

        static_for<0, BN / 32>([&](auto nb_c) {
            constexpr int nb = decltype(nb_c)::value;
            if (nb ? skip1 : skip0) return;
            bf16x8 dsf0[2], dsf1[2];
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                dsf0[jj] = TS::tr_frag(Sbuf(cur, 0), sbase, 32 * nb + 16 * jj, 32 * w);
                dsf1[jj] = TS::tr_frag(Sbuf(cur, 1), sbase, 32 * nb + 16 * jj, 32 * w);
            }
            auto pace_hook = [&](auto idx) {
                constexpr int m = decltype(idx)::value;
                if constexpr (m % kEvery == kEvery - 1) {
                    constexpr int run = m / kEvery;
                    if constexpr (nb == 0) {
                        sk.template issue_one<run>(ksrc, kdst, w, k_lim, ksb);
                    } else if constexpr (run < decltype(ss)::PER) {
                        ss.template issue_one<run>(s0src, s0dst, w, s_lim, kTile * 2);
                    } else {
                        ss.template issue_one<run - decltype(ss)::PER>(s1src, s1dst, w, s_lim, kTile * 2);
                    }
                }
            };
            trfrag_gemm_dual<D, 2, kBPipe>(lds_addr(Kbuf(cur)) + tbase + (uint32_t)(32 * nb * TL::kPitch), dsf0, dsf1, acc0, acc1, pace_hook);
        });
    }

    __syncthreads();
    mfma_fence();
    {
        constexpr int kPitchO = D * 2 + 16;
        __bf16* ob = (__bf16*)a.dq.ptr + b * a.dq.stride_b + h0 * a.dq.stride_h;
        store_tile_T<D>(lds0 + w * 32 * kPitchO, acc0, a.scale, ob, a.dq.stride_s, qw_lo, a.S, lane);
        store_tile_T<D>(lds0 + w * 32 * kPitchO, acc1, a.scale, ob + a.dq.stride_h, a.dq.stride_s, qw_lo, a.S, lane);
    }
}

template <int D, bool HAS_DOC>
__global__ __launch_bounds__(kBwdThreads, 1) void attn_bwd_dq_ds_pair_bf16_kernel(AttnArgs a) {
    attn_bwd_dq_ds_pair_bf16_item<D, HAS_DOC>(fresh_args(), (int)blockIdx.x);
}

template <typename K>
static int opt_in_lds(K kernel, size_t bytes, const char* name) {
    if (bytes <= 64 * 1024) return MA_OK;
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return fail(MA_ERR_LAUNCH, "hipFuncSetAttribute(%s, %zu): %s", name, bytes, hipGetErrorString(e));
    return MA_OK;
}

template <int D, bool HAS_DOC>
static int bwd_dd(const AttnArgs& a, hipStream_t st) {
    constexpr int RPB = 256 / (D / 8);
    const int64_t nrows = (int64_t)a.B * a.Hq * a.S;
    int rc = MA_OK;
    const bool hand_over = a.ds != nullptr;  // dS^T goes from the dK/dV kernel to the dQ kernel through a.ds
    // delta on its own when the dQ stage, which computes it for its own rows, is not asked for, and
    // always with the hand-over (its dQ kernel reads neither O nor dO)
    if ((a.stages & MA_BWD_DELTA) && (hand_over || !(a.stages & MA_BWD_DQ))) {
        hipLaunchKernelGGL(attn_delta_bf16_kernel<D>, dim3((unsigned)((nrows + RPB - 1) / RPB)), dim3(256), 0, st, a);
        rc = check_launch("attn_delta_bf16_kernel");
        if (rc) return rc;
    }
    const size_t lds_kv = (size_t)4 * Tile<D>::bytes(kStep) + 2 * kStep * (4 + 4 + 8) + 16 + (kBwdThreads / 64) * 512;  // + work-queue box, step tables
    if (hand_over) {
        if (a.stages & MA_BWD_DKV) {
            rc = opt_in_lds(attn_bwd_dkv_bf16_kernel<D, HAS_DOC, true>, lds_kv, "attn_bwd_dkv_bf16");
            if (rc) return rc;
            static const int resident = resident_workgroups(attn_bwd_dkv_bf16_kernel<D, HAS_DOC, true>, kBwdThreads, lds_kv);
            hipLaunchKernelGGL((attn_bwd_dkv_bf16_kernel<D, HAS_DOC, true>), dim3(queue_grid(work_grid(a.B * a.T, a.Hkv, 1), a.map.work_counters, resident), 1, 1),
                               dim3(kBwdThreads), lds_kv, st, a);
            rc = check_launch("attn_bwd_dkv_bf16_kernel");
            if (rc) return rc;
        }
        const int G = a.Hq / a.Hkv;
        if ((a.stages & MA_BWD_DQ) && G % 2 == 0 && D >= MA_DQ_PAIR_MIN_D) {
            const size_t lds_q = (size_t)2 * (Tile<D>::bytes(kStep) + 2 * Tile<kTile>::bytes(kStep)) + 16 + (kBwdThreads / 64) * 512;
            rc = opt_in_lds(attn_bwd_dq_ds_pair_bf16_kernel<D, HAS_DOC>, lds_q, "attn_bwd_dq_ds_pair_bf16");
            if (rc) return rc;
            hipLaunchKernelGGL((attn_bwd_dq_ds_pair_bf16_kernel<D, HAS_DOC>), dim3(work_grid(a.B * a.T, a.Hkv, G / 2), 1, 1), dim3(kBwdThreads),
                               lds_q, st, a);
            rc = check_launch("attn_bwd_dq_ds_pair_bf16_kernel");
        } else if (a.stages & MA_BWD_DQ) {
            const size_t lds_q = (size_t)2 * Tile<D>::bytes(kStep) + 2 * Tile<kTile>::bytes(kStep) + 16 + (kBwdThreads / 64) * 512;
            const size_t lds_store = (size_t)(kBwdThreads / 64) * 32 * (D * 2 + 16);   // the epilogue's scratch
            const size_t lds = lds_q > lds_store ? lds_q : lds_store;
            rc = opt_in_lds(attn_bwd_dq_ds_bf16_kernel<D, HAS_DOC>, lds, "attn_bwd_dq_ds_bf16");
            if (rc) return rc;
            hipLaunchKernelGGL((attn_bwd_dq_ds_bf16_kernel<D, HAS_DOC>), dim3(work_grid(a.B * a.T, a.Hkv, a.Hq / a.Hkv), 1, 1), dim3(kBwdThreads),
                               lds, st, a);
            rc = check_launch("attn_bwd_dq_ds_bf16_kernel");
        }
        return rc;
    }
    if (a.stages & MA_BWD_DQ) {  // first: the dK/dV kernel reads the delta this one may be writing
        const size_t lds_q = (size_t)4 * Tile<D>::bytes(kStep) + 2 * kStep * 8 + 16 + (kBwdThreads / 64) * 256;  // K/V ring, kv document ids, step tables
        rc = opt_in_lds(attn_bwd_dq_bf16_kernel<D, HAS_DOC>, lds_q, "attn_bwd_dq_bf16");
        if (rc) return rc;
        hipLaunchKernelGGL((attn_bwd_dq_bf16_kernel<D, HAS_DOC>), dim3(work_grid(a.B * a.T, a.Hkv, a.Hq / a.Hkv), 1, 1), dim3(kBwdThreads),
                           lds_q, st, a);
        rc = check_launch("attn_bwd_dq_bf16_kernel");
        if (rc) return rc;
    }
    if (a.stages & MA_BWD_DKV) {
        rc = opt_in_lds(attn_bwd_dkv_bf16_kernel<D, HAS_DOC, false>, lds_kv, "attn_bwd_dkv_bf16");
        if (rc) return rc;
        static const int resident = resident_workgroups(attn_bwd_dkv_bf16_kernel<D, HAS_DOC, false>, kBwdThreads, lds_kv);
        hipLaunchKernelGGL((attn_bwd_dkv_bf16_kernel<D, HAS_DOC, false>), dim3(queue_grid(work_grid(a.B * a.T, a.Hkv, 1), a.map.work_counters, resident), 1, 1), dim3(kBwdThreads), lds_kv,
                           st, a);
        rc = check_launch("attn_bwd_dkv_bf16_kernel");
    }
    return rc;
}

template <int D>
static int bwd_d(const AttnArgs& a, hipStream_t st) {
    return a.doc ? bwd_dd<D, true>(a, st) : bwd_dd<D, false>(a, st);
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
