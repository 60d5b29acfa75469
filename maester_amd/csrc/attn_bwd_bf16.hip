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

namespace ma {

#ifdef MA_TICKS
// measurement builds only (maester_amd/kernel_ticks.py): cycles a wave spends between two of the marks
// MA_TICK(n) of the dK/dV kernel; in the library the marks compile to nothing
__device__ unsigned long long ma_dbg_ticks[4];
struct Ticks {
    unsigned long long begin = 0, acc = 0;
    unsigned n = 0;
    bool armed = false;
    template <int ID>
    __device__ __forceinline__ void at() {
        if constexpr (ID == MA_T_END) {
            if (armed) { acc += __builtin_readcyclecounter() - begin; ++n; armed = false; }
        }
        if constexpr (ID == MA_T_BEGIN) { begin = __builtin_readcyclecounter(); armed = true; }
    }
};
#define MA_TICK(id) ticks.template at<id>()
#else
#define MA_TICK(id)
#endif

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
    // all rows leave LDS first, then go out (one LDS round trip; 32-bit offsets from a uniform base)
    MA_GLB char* g0 = (MA_GLB char*)(gbase + (int64_t)row0 * stride);
    const uint32_t row_bytes = (uint32_t)(stride * 2);
    u32x4 val[32 / RPI];
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) val[it] = *(MA_LDS u32x4*)(scratch + (it * RPI + rsub) * kPitchO + c * 16);
    if (row0 + 31 < rows_end) {
#pragma unroll
        for (int it = 0; it < 32 / RPI; ++it) *(MA_GLB u32x4*)(g0 + (uint32_t)(it * RPI + rsub) * row_bytes + c * 16) = val[it];
    } else {
#pragma unroll
        for (int it = 0; it < 32 / RPI; ++it)
            if (row0 + it * RPI + rsub < rows_end) *(MA_GLB u32x4*)(g0 + (uint32_t)(it * RPI + rsub) * row_bytes + c * 16) = val[it];
    }
}

// ------------------------------------------------------------------------------------------------
// delta[b,h,q] = sum_d O[b,q,h,d] * dO[b,q,h,d]
// ------------------------------------------------------------------------------------------------
// A pure read stream (O and dO once, 2 * elt * B*S*Hq*D bytes): every thread has the loads of kDeltaRows rows
// in flight before it adds anything up.
constexpr int kDeltaRows = 4;
template <int D>
__global__ __launch_bounds__(256) void attn_delta_bf16_kernel(AttnArgs a) {
    constexpr int LPR = D / 8;  // lanes per row
    constexpr int RPB = 256 / LPR;
    const int sub = threadIdx.x % LPR;
    const int64_t nrows = (int64_t)a.B * a.Hq * a.S;
    const int64_t row0 = (int64_t)blockIdx.x * (RPB * kDeltaRows) + threadIdx.x / LPR;
    bf16x8 x[kDeltaRows], y[kDeltaRows];
#pragma unroll
    for (int i = 0; i < kDeltaRows; ++i) {
        const int64_t row = min(row0 + i * RPB, nrows - 1);      // (rows past the end re-read the last one; not written)
        const int q = row % a.S;
        const int h = (row / a.S) % a.Hq;
        const int b = row / ((int64_t)a.S * a.Hq);
        const __bf16* op = (const __bf16*)a.o.ptr + b * a.o.stride_b + (int64_t)q * a.o.stride_s + h * a.o.stride_h;
        const __bf16* gp = (const __bf16*)a.dout.ptr + b * a.dout.stride_b + (int64_t)q * a.dout.stride_s + h * a.dout.stride_h;
        x[i] = __builtin_nontemporal_load((const bf16x8*)(op + sub * 8));   // O is not read again in this step (dO is, at once)
        y[i] = *(const bf16x8*)(gp + sub * 8);
    }
#pragma unroll
    for (int i = 0; i < kDeltaRows; ++i) {
        float acc = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc += (float)x[i][e] * (float)y[i][e];
#pragma unroll
        for (int off = LPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
        const int64_t row = row0 + i * RPB;
        if (row < nrows && sub == 0) a.delta[row] = acc;
    }
}

// ------------------------------------------------------------------------------------------------
// dK / dV
// ------------------------------------------------------------------------------------------------
// The q-side steps of one dK/dV work item, resolved ahead of the loop that runs them.  A wave that has
// its SIMD to itself pays four cycles for every instruction it issues between two MFMA chains, so
// whatever a step needs is worked out 64 steps at a time, one candidate step per lane, and kept as a
// record of ready-made addresses in the wave's own slice of LDS; taking a step is then three
// broadcast LDS reads and a dozen v_readfirstlane.
//   word 0       first q row | query head within the group << 24 | act1 << 29 | act0 << 30 | partial << 31
//   word 1       rows of the step that lie inside the sequence (1 .. 64)
//                (act0 / act1: this wave has something to do in the first / second 32-row block)
//   words 2,3    address of the step's first Q row        words 4,5    of its first dO row
//   words 6,7    of its first lse entry                   words 8,9    of its first delta entry
//   words 10,11  of its dS^T slab in the workspace (WRITE_DS)
// Every wave of a workgroup derives the same sequence of steps (same inputs); only the two block
// bits are its own.  Nothing a refill needs is kept between refills except the position in the walk:
// it is derived again from the argument block, so that the step loop holds no registers for it.
// Which chain of a step carries which of the next step's tile loads, in eighths of a wave's runs:
// kDkvPlan[block][chain (0: S / dP, 1: dV / dK)] = {tile (0: Q, 1: dO), first eighth, eighths}.
// The Q tile rides in the first block's S / dP chain, the dO tile in the second block's: both in the first
// block, or split over more chains, measured slower.
constexpr int kDkvPlan[2][2][3] = {{{0, 0, 8}, {0, 0, 0}}, {{1, 0, 8}, {0, 0, 0}}};
constexpr int kDkvRecWords = 12;
constexpr int kDkvRecBytes = 64 * kDkvRecWords * 4;  // LDS per wave
template <bool HAS_DOC, bool WRITE_DS>
struct DkvSteps {
    MA_LDS uint32_t* tab;
    int cbase, cnt, pos;
    __device__ __forceinline__ void start(MA_LDS uint32_t* table) { tab = table; cbase = 0; cnt = 0; pos = -1; }

    // the next candidates that hold a step at all; false when the walk is over.
    // FIRST (an item's first fill): the candidates are scanned at least once, and `mid1` / `mid2` run
    // while the scan's two dependent loads (list entries, then id ranges and workspace slots) are on
    // their way -- the item's own operand loads go there, so that the round trips do not queue up behind
    // them.  Every load of the scan is unconditional (a load under a condition is waited for on the spot).
    template <bool FIRST, class F1, class F2>
    __device__ __forceinline__ bool refill(const int j, const int hk, const int b, const int w, F1&& mid1, F2&& mid2) {
        KernArgs& a = fresh_args();
        const int lane = __lane_id();
        const int G = a.Hq / a.Hkv;
        const size_t mrow = (size_t)b * a.T + j;
        const bool use_rng = HAS_DOC && a.map.block_doc_range != nullptr;
        const int64_t* rng = use_rng ? a.map.block_doc_range + (size_t)b * (2 * ((a.S + 63) / 64)) * 2 : nullptr;
        DocRange own;  // id range of the wave's own kv rows: in the same round trip as the list lengths
        int np, nf;
        if (use_rng) scalar_load2_range(a.map.q_num_blocks + mrow, a.map.full_q_num_blocks + mrow,
                                        rng + (size_t)(min(j * kTile + 32 * w, a.S - 1) / MA_DOC_BLOCK) * 2, np, nf, own);
        else scalar_load2(a.map.q_num_blocks + mrow, a.map.full_q_num_blocks + mrow, np, nf);
        const int n = np + nf, per_pass = n * (kTile / kStep), total = per_pass * G;
        const bool bounded = a.causal || a.window >= 0, windowed = a.window >= 0;
        const int wlim = windowed ? (int)min(a.window, (int64_t)0x3fffffff) : 0x7fffffff;
        const int kw_lo = j * kTile + 32 * w, kw_hi = kw_lo + 31;
        int vis_lo, vis_hi, blk_lo, blk_hi;
        visibility_limits(true, j * kTile, j * kTile + kTile - 1, kStep, bounded, wlim, windowed, vis_lo, vis_hi);
        visibility_limits(true, kw_lo, kw_hi, 32, bounded, wlim, windowed, blk_lo, blk_hi);
        int64_t own_lo = 0, own_hi = 0;
        if (use_rng) {
            own_lo = own.lo();
            own_hi = own.hi();
        }
        const int32_t* pl = a.map.q_indices + mrow * a.T;
        const int32_t* fl = a.map.full_q_indices + mrow * a.T;
        const void* kbase = (const void*)((const __bf16*)a.k.ptr + b * a.k.stride_b + hk * a.k.stride_h);  // readable, at least a row long
        cnt = 0;
        auto scan = [&](auto first_c) {
            constexpr bool first = decltype(first_c)::value;
            const int c = cbase + lane;
            const bool valid = (c < total) & (n > 0);
            const int cc = valid ? c : 0;
            const int rep = cc / max(per_pass, 1), wi = cc - rep * per_pass;
            const int it = wi / (kTile / kStep), half = wi - it * (kTile / kStep);
            const int idx = max(n - 1 - it, 0);  // from the last q tile down: the workgroups of a document start on the same tiles
            const bool partial = idx < np;
            const int32_t* entry = partial ? pl + idx : fl + (idx - np);  // (no candidate: the first entry of a list, unused)
            int tile = *(const MA_GLB int32_t*)entry;
            if constexpr (first) {
                asm volatile("" ::: "memory");
                mid1();
                asm volatile("" ::: "memory");
            }
            tile = valid ? tile : 0;
            const int r0 = tile * kTile + half * kStep;
            const bool vis = valid & (r0 < a.S) & (!partial | ((r0 >= vis_lo) & (r0 <= vis_hi)));
            bool act0 = (r0 < a.S) & (!partial | ((r0 >= blk_lo) & (r0 <= blk_hi)));
            bool act1 = (r0 + 32 < a.S) & (!partial | ((r0 + 32 >= blk_lo) & (r0 + 32 <= blk_hi)));
            // what depends on the tile's number goes out together: the id ranges of the step's two blocks
            // and the tile's slot in the dS workspace.  Where there is nothing to look up (no range table,
            // a full tile, no step) the range load reads the head of the K tensor and its result is not used.
            uint32_t tslot = 0;
            // (clamped to the workspace: a count that is stale or too small -- it comes from the host -- must not
            // turn into a store past the end; the gradients of such a call are undefined, memory is not)
            if constexpr (WRITE_DS) tslot = min((uint32_t)((const MA_GLB int32_t*)a.map.tile_slot)[((int64_t)b * a.T + tile) * a.T + j], (uint32_t)(a.ds_tiles - 1));
            i64x2 e0 = {0, 0}, e1 = {0, 0};
            bool look = false;
            if constexpr (HAS_DOC) {
                look = use_rng & partial & vis;
                const MA_GLB i64x2* e = (const MA_GLB i64x2*)(look ? (const void*)(rng + (size_t)(r0 / 32) * 2) : kbase);
                e0 = e[0];
                e1 = e[1];
            }
            if constexpr (first) {
                asm volatile("" ::: "memory");
                mid2();
                asm volatile("" ::: "memory");
            }
            if constexpr (HAS_DOC) {  // no row of the block shares a document with the wave's own rows
                act0 &= !look | ((e0[0] <= own_hi) & (e0[1] >= own_lo));
                act1 &= !look | ((e1[0] <= own_hi) & (e1[1] >= own_lo));
            }
            const uint64_t mask = __ballot(vis);
            const int at = __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
            if (vis) {
                const int h = hk * G + rep;
                const uint64_t qa = (uint64_t)((const __bf16*)a.q.ptr + b * a.q.stride_b + h * a.q.stride_h + (int64_t)r0 * a.q.stride_s);
                const uint64_t ga = (uint64_t)((const __bf16*)a.dout.ptr + b * a.dout.stride_b + h * a.dout.stride_h + (int64_t)r0 * a.dout.stride_s);
                const size_t row = ((size_t)b * a.Hq + h) * a.S + r0;
                const uint64_t la = (uint64_t)(a.lse + row), ea = (uint64_t)(a.delta + row);
                uint64_t da = 0;
                if (WRITE_DS) {
                    da = (uint64_t)((char*)a.ds + ((uint64_t)(uint32_t)h * (uint64_t)a.ds_tiles + tslot) * (kTile * kTile * 2) + (r0 & (kTile - 1)) * 2);
                }
                MA_LDS uint32_t* rec = tab + at * kDkvRecWords;
                *(MA_LDS u32x4*)rec = u32x4{(uint32_t)r0 | ((uint32_t)rep << 24) | ((uint32_t)act1 << 29) | ((uint32_t)act0 << 30) | ((uint32_t)partial << 31),
                                            (uint32_t)min(kStep, a.S - r0), (uint32_t)qa, (uint32_t)(qa >> 32)};
                *(MA_LDS u32x4*)(rec + 4) = u32x4{(uint32_t)ga, (uint32_t)(ga >> 32), (uint32_t)la, (uint32_t)(la >> 32)};
                *(MA_LDS u32x4*)(rec + 8) = u32x4{(uint32_t)ea, (uint32_t)(ea >> 32), (uint32_t)da, (uint32_t)(da >> 32)};
            }
            cbase += 64;
            cnt = __builtin_popcountll(mask);
        };
        if constexpr (FIRST) scan(std::true_type{});
        while (cnt == 0 && cbase < total) scan(std::false_type{});
        pos = 0;
        return cnt != 0;
    }
    // moves on to the next step: false when the walk is over
    __device__ __forceinline__ bool advance(const int j, const int hk, const int b, const int w) {
        if (++pos < cnt) return true;
        return refill<false>(j, hk, b, w, [] {}, [] {});
    }
    // the first step of an item (call after start())
    template <class F1, class F2>
    __device__ __forceinline__ bool advance_first(const int j, const int hk, const int b, const int w, F1&& mid1, F2&& mid2) {
        return refill<true>(j, hk, b, w, mid1, mid2);
    }
};
__device__ __forceinline__ uint64_t uniform64(uint32_t lo, uint32_t hi) {
    return (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane(lo) | ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane(hi) << 32);
}

// WRITE_DS: every 32 x 32 block that a wave works on also leaves its dS^T in a.ds, for the dQ kernel that only
// multiplies it with K.  A block that the wave skips is not written, and the dQ kernel never uses it: both
// kernels decide per 32 x 32 block (32 q rows of one wave there, 32 kv rows of one wave here) by the same three
// tests -- the tile is partial and (a) the largest q row lies below the smallest kv row, or (b) the smallest q row
// lies more than the window above the largest kv row, or (c) the document-id ranges of the two row blocks
// (block_doc_range) are disjoint -- so a block is skipped on both sides or on neither.  (Blocks of q rows past the
// end of the sequence are skipped here only; there the dQ kernel computes columns that it never stores.)
template <int D, bool HAS_DOC, bool WRITE_DS, bool FULL>
__device__ __forceinline__ void attn_bwd_dkv_bf16_item(KernArgs& a, const int wg_id
#ifdef MA_TICKS
    , Ticks& ticks
#endif
) {
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
    const int kw_lo = j * kTile + 32 * w;
    const int kv = kw_lo + r;
    const bool kvalid = kv < a.S;
    const bool bounded = a.causal || a.window >= 0;
    const float sl2 = a.scale * kLog2e;
    const float neg_inv_scale = -1.0f / a.scale;
    const int S = a.S;

    const __bf16* kp = (const __bf16*)a.k.ptr + b * a.k.stride_b + hk * a.k.stride_h;
    const __bf16* vp = (const __bf16*)a.v.ptr + b * a.v.stride_b + hk * a.v.stride_h;
    const int64_t* drow = HAS_DOC ? a.doc + (size_t)b * S : nullptr;
    const int kvc = min(kv, S - 1);
    const int64_t dock = HAS_DOC ? drow[kvc] : 0;
    const int wlim = a.window >= 0 ? (int)min(a.window, (int64_t)0x3fffffff) : 0x7fffffff;

    // K and V rows of the wave go straight from global memory into MFMA operand fragments (lane (r, hh):
    // elements 16*kk + 8*hh .. +7 of row kw_lo + r, one 16-byte load each; rows past the end of the
    // sequence re-read the last valid row and are masked).  Nothing waits for them here: the walk is
    // resolved and the first tiles are requested while they are on their way.
    bf16x8 kf[KK], vf[KK];
    const __bf16* krow = kp + (int64_t)kvc * a.k.stride_s + 8 * hh;
    const __bf16* vrow = vp + (int64_t)kvc * a.v.stride_s + 8 * hh;
    auto load_kf = [&]() {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) kf[kk] = *(const bf16x8*)(krow + 16 * kk);
    };
    auto load_vf = [&]() {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) vf[kk] = *(const bf16x8*)(vrow + 16 * kk);
    };

    f32x16 dkacc[DB], dvacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) dkacc[db][v] = dvacc[db][v] = 0.f;

    DkvSteps<HAS_DOC, WRITE_DS> st;
    st.start((MA_LDS uint32_t*)(aux + 2 * BM * (4 + 4 + 8) + 16) + w * (kDkvRecBytes / 4));

    // The Q and dO tiles have the same shape: one set of slots.  Every wave moves the same number of runs
    // of a tile from inside its MFMA chains (kPaced, one every four MFMAs); the run that is left over
    // (a tile is 4 * kPaced + 1 runs) is moved by wave 0 (Q) or wave 1 (dO) when the step begins.
    using SQ = DirectStager<D, BM, NW>;
    constexpr int kPaced = (SQ::NL - 1) / NW;
    static_assert(SQ::NL == NW * kPaced + 1 && (2 * KK) % kPaced == 0, "tile runs per wave");
    const uint32_t qsb = (uint32_t)(a.q.stride_s * 2), gsb = (uint32_t)(a.dout.stride_s * 2);  // row strides in bytes
    // the lane's byte offset into a Q tile and into a dO tile for each of its runs (the two tensors may have
    // different row strides), and for the left-over run of the tile its wave moves
    uint32_t qoff[kPaced], goff[kPaced], off_last;
    {
        int row, chunk;
#pragma unroll
        for (int p = 0; p < kPaced; ++p) {
            SQ::slot(w + p * NW, lane, row, chunk);
            qoff[p] = (uint32_t)row * qsb + (uint32_t)chunk * 16u;
            goff[p] = (uint32_t)row * gsb + (uint32_t)chunk * 16u;
        }
        SQ::slot(SQ::NL - 1, lane, row, chunk);
        off_last = (uint32_t)row * (w == 0 ? qsb : gsb) + (uint32_t)chunk * 16u;
    }
    constexpr uint32_t kRowBytes = D * 2;
    // Where a run comes from.  FULL (the sequence is a whole number of steps, so every tile has all of its
    // rows): the tile's address, and a run is a plain load into LDS -- on the last step of a walk, when there
    // is no next tile, the address stays on the current one, which is read once more.  Otherwise: a buffer
    // descriptor of the tile with `rows` rows in range; lanes of rows past it (all of them when there is no
    // next tile) read nothing and zeros land in LDS.  (The plain load is the faster instruction here.)
    struct Src { uint64_t at; u32x4 rsrc; };
    auto tile_src = [&](uint64_t at, int rows, uint32_t stride_bytes) {
        Src t{at, u32x4{0, 0, 0, 0}};
        if constexpr (!FULL) t.rsrc = tile_rsrc(at, rows > 0 ? (uint32_t)(rows - 1) * stride_bytes + kRowBytes : 0u);
        return t;
    };
    auto run_to_lds = [&](const Src& t, uint32_t off, uint32_t lds) {
        if constexpr (FULL) global_to_lds_run((const void*)t.at, off, lds);
        else buffer_to_lds_run(t.rsrc, off, lds);
    };
    auto run_to_lds_at = [&](const Src& t, uint32_t off, uint32_t lds_base, auto imm_c) {
        if constexpr (FULL) global_to_lds_run_at<decltype(imm_c)::value>((const void*)t.at, off, lds_base);
        else buffer_to_lds_run_at<decltype(imm_c)::value>(t.rsrc, off, lds_base);
    };
    // a whole tile at once (the first step of an item)
    auto burst = [&](const Src& t, const uint32_t* off, uint32_t dst, bool with_last) {
#pragma unroll
        for (int p = 0; p < kPaced; ++p) run_to_lds(t, off[p], dst + (w + p * NW) * 1024);
        if (with_last) run_to_lds(t, off_last, dst + (SQ::NL - 1) * 1024);
    };
    // per-row lse / delta / document id of a step: loaded for the step after the current one, written
    // to LDS when that step begins by wave 1 (lse), wave 2 (delta) and wave 3 (ids).  Every wave issues
    // both loads, each from the array it is in charge of (no branch: a conditional load would be waited
    // for on the spot, to merge its result with the value carried otherwise).
    float row_f = 0.f;
    int64_t row_d = 0;
    auto load_rows = [&](uint64_t lse_at, uint64_t delta_at, int r0, int rows) {
        const int li = min(lane, rows - 1);
        const MA_GLB float* fsrc = (const MA_GLB float*)(w == 2 ? delta_at : lse_at);
        row_f = fsrc[li];
        if (HAS_DOC) row_d = ((const MA_GLB int64_t*)drow)[r0 + li];
    };
    // the step the loop stands on, and the one after it
    uint32_t nflags = 0;
    uint64_t ds_at = 0, nds_at = 0, nq_at = 0, ng_at = 0;
    // (the fields of the current step's word are carried as variables of their own: decoded from the word
    // inside the loop, the compiler splits the accumulators' live ranges around the skipped-block path
    // and spills them)
    int q0 = 0;
    bool partial = false, act0 = false, act1 = false;
    auto decode = [&](uint32_t word) {
        q0 = (int)(word & 0xffffffu);
        partial = (word >> 31) != 0;
        act0 = (word >> 30) & 1u;
        act1 = (word >> 29) & 1u;
    };
    bool have = st.advance_first(j, hk, b, w, load_kf, load_vf);
    if (have) {
        MA_LDS uint32_t* rec = st.tab + st.pos * kDkvRecWords;
        const u32x4 x0 = *(MA_LDS u32x4*)rec, x1 = *(MA_LDS u32x4*)(rec + 4), x2 = *(MA_LDS u32x4*)(rec + 8);
        const uint32_t flags = __builtin_amdgcn_readfirstlane(x0[0]);
        nq_at = uniform64(x0[2], x0[3]);
        ng_at = uniform64(x1[0], x1[1]);
        ds_at = uniform64(x2[2], x2[3]);
        decode(flags);
        const int r0 = q0;
        const int rows = (int)__builtin_amdgcn_readfirstlane(x0[1]);
        burst(tile_src(nq_at, rows, qsb), qoff, lds_addr(Qbuf(0)), w == 0);
        burst(tile_src(ng_at, rows, gsb), goff, lds_addr(Gbuf(0)), w == 1);
        load_rows(uniform64(x1[2], x1[3]), uniform64(x2[0], x2[1]), r0, rows);
    }
    const uint32_t ds_lane = (uint32_t)((32 * w + r) * (kTile * 2) + 16 * hh);

    for (int n = 0; have; ++n) {
        MA_TICK(0);
        const int cur = n & 1;
        const lds_ptr Qs = Qbuf(cur), Gs = Gbuf(cur);
        MA_LDS float* lse2s = Lbuf(cur);
        MA_LDS float* dls = Ebuf(cur);
        MA_LDS int64_t* qdoc = Dbuf(cur);
        if (w == 1) lse2s[lane] = row_f * neg_inv_scale;  // -lse / scale: the addend of S
        if (w == 2) dls[lane] = -row_f;                    // -delta: the addend of dP
        if (HAS_DOC && w == 3) qdoc[lane] = row_d;
        const bool have_next = st.advance(j, hk, b, w);
        u32x4 x0 = {0, 0, 0, 0}, x1 = x0, x2 = x0;
        if (have_next) {  // the record of the next step: read now, picked up behind the barrier
            MA_LDS uint32_t* rec = st.tab + st.pos * kDkvRecWords;
            x0 = *(MA_LDS u32x4*)rec;
            x1 = *(MA_LDS u32x4*)(rec + 4);
            x2 = *(MA_LDS u32x4*)(rec + 8);
        }
        wait_vmem();
        MA_TICK(20);
        __syncthreads();
        MA_TICK(1);

        const int cq0 = q0;
        const bool cpartial = partial;
        const bool skip[BM / 32] = {!act0, !act1};  // blocks in which this wave has nothing to do
        MA_GLB char* ds_out = (MA_GLB char*)ds_at;  // (a global pointer: a generic one would make the stores flat ones, counted with the LDS reads)
        // The tile loads of the next step are spread over the chains of this step's first 32-row block,
        // one run every four MFMAs (Q tile from the S / dP chain, dO tile from the dV / dK chain): issued
        // in one burst they fill the memory pipeline and stall the wave with the matrix cores idle, and
        // issued later in the step they have not landed when the next step begins.
        int nrows = 0;  // (the last step of a walk: see run_to_lds)
        if (have_next) {
            nflags = __builtin_amdgcn_readfirstlane(x0[0]);
            nq_at = uniform64(x0[2], x0[3]);
            ng_at = uniform64(x1[0], x1[1]);
            nds_at = uniform64(x2[2], x2[3]);
            const int nr0 = (int)(nflags & 0xffffffu);
            nrows = (int)__builtin_amdgcn_readfirstlane(x0[1]);  // (from the record: the sequence length is not kept in a register)
            load_rows(uniform64(x1[2], x1[3]), uniform64(x2[0], x2[1]), nr0, nrows);
        }
        const Src qsrc = tile_src(nq_at, nrows, qsb), gsrc = tile_src(ng_at, nrows, gsb);
        if (have_next) {
            if (w == 0) run_to_lds(qsrc, off_last, lds_addr(Qbuf(cur ^ 1)) + (SQ::NL - 1) * 1024);
            if (w == 1) run_to_lds(gsrc, off_last, lds_addr(Gbuf(cur ^ 1)) + (SQ::NL - 1) * 1024);
        }
        const uint32_t qdst = lds_addr(Qbuf(cur ^ 1)) + w * 1024, gdst = lds_addr(Gbuf(cur ^ 1)) + w * 1024;  // the wave's first run

        // The two 32-row blocks of the step are two copies of the same code (mb is a compile-time
        // constant in each), so that each chain carries exactly the loads planned for it.
        auto block = [&](auto mb_c) {
            constexpr int mb = decltype(mb_c)::value;
            MA_TICK(2);
            const int qb0 = cq0 + 32 * mb;
            // which runs of which tile (0: Q, 1: dO) the block's two chains move: {tile, first run, runs}
            constexpr int kPlanA[3] = {kDkvPlan[mb][0][0], kDkvPlan[mb][0][1] * kPaced / 8, kDkvPlan[mb][0][2] * kPaced / 8};
            constexpr int kPlanB[3] = {kDkvPlan[mb][1][0], kDkvPlan[mb][1][1] * kPaced / 8, kDkvPlan[mb][1][2] * kPaced / 8};
            auto move_run = [&](auto tile_c, auto run_c) {
                constexpr int run = decltype(run_c)::value;
                if constexpr (decltype(tile_c)::value == 0)
                    run_to_lds_at(qsrc, qoff[run], qdst, std::integral_constant<int, run * (NW * 1024)>{});
                else
                    run_to_lds_at(gsrc, goff[run], gdst, std::integral_constant<int, run * (NW * 1024)>{});
            };
            if (skip[mb]) {
                // (nothing is left in the dS workspace for a block the wave skips: the dQ kernel skips the same
                // 32 x 32 blocks -- see the note on WRITE_DS above the kernel)
                if (have_next) {  // the loads its chains would have carried
                    static_for<0, kPlanA[2]>([&](auto r) { move_run(std::integral_constant<int, kPlanA[0]>{}, std::integral_constant<int, kPlanA[1] + decltype(r)::value>{}); });
                    static_for<0, kPlanB[2]>([&](auto r) { move_run(std::integral_constant<int, kPlanB[0]>{}, std::integral_constant<int, kPlanB[1] + decltype(r)::value>{}); });
                }
                return;
            }
            auto a_hook = [&](auto idx) {
                constexpr int i = decltype(idx)::value;
                if constexpr (kPlanA[2] > 0) {
                    constexpr int every = (2 * KK) / kPlanA[2];
                    if constexpr (i % every == every - 1) move_run(std::integral_constant<int, kPlanA[0]>{}, std::integral_constant<int, kPlanA[1] + i / every>{});
                }
            };
            auto b_hook = [&](auto idx) {
                constexpr int i = decltype(idx)::value;
                if constexpr (kPlanB[2] > 0) {
                    constexpr int every = (2 * KK) / kPlanB[2];
                    if constexpr (i % every == every - 1) move_run(std::integral_constant<int, kPlanB[0]>{}, std::integral_constant<int, kPlanB[1] + i / every>{});
                }
            };

            // S = Q K^T and dP = dO V^T for 32 q rows x the wave's 32 kv rows (lane owns one kv row)
            // The accumulators start from -lse / scale and -delta of their q rows (an element's row is
            // 8 * (v / 4) + 4 * hh + v % 4), read from LDS straight into them: the chain then leaves
            // S - lse / scale and dP - delta, and neither is touched by the vector ALU for it.
            f32x16 s, dp;
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const f32x4 l4 = *(MA_LDS f32x4*)(lse2s + 32 * mb + 8 * g4 + 4 * hh);
                const f32x4 e4 = *(MA_LDS f32x4*)(dls + 32 * mb + 8 * g4 + 4 * hh);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    s[4 * g4 + e] = l4[e];
                    dp[4 * g4 + e] = e4[e];
                }
            }
            const uint32_t roff = (uint32_t)(32 * mb * TL::kPitch);
            // The two products run one after the other so that the exponentials of S (a quarter-rate
            // instruction each) are taken in the shadow of the dP MFMAs: one value per MFMA, from the
            // second MFMA after S is complete; what does not fit follows the chain.
            constexpr int kFirstExp = KK + 2, kHooked = (2 * KK - kFirstExp) < 16 ? (2 * KK - kFirstExp) : 16;
            auto chain_hook = [&](auto idx) {
                constexpr int i = decltype(idx)::value;
                a_hook(idx);
                if constexpr (i >= kFirstExp && i - kFirstExp < 16) s[i - kFirstExp] = fast_exp2(s[i - kFirstExp] * sl2);
            };
            rowfrag_gemm2<D, kBPipe, false, false, decltype(chain_hook)&, true, true>(lds_addr(Qs) + rbase + roff, kf, s, lds_addr(Gs) + rbase + roff, vf, dp, chain_hook);
#pragma unroll
            for (int v = kHooked; v < 16; ++v) s[v] = fast_exp2(s[v] * sl2);
            MA_TICK(3);

            bf16x8 pf[2], dsf[2];
            // d = q - kv for element v is drel + 8*(v/4) + v%4; range test as one unsigned compare
            const int drel = qb0 + 4 * hh - kv;
            const int dlo = bounded ? 0 : -0x40000000;
            const int dhi = min(wlim, S - 1 - kv);              // q - kv <= window, q < S
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
                    i64x2 ida = {0, 0}, idb = {0, 0};
                    if (HAS_DOC && MASKED) {
                        ida = *(MA_LDS i64x2*)(qdoc + qoff);
                        idb = *(MA_LDS i64x2*)(qdoc + qoff + 2);
                    }
                    const int64_t ids[4] = {ida[0], ida[1], idb[0], idb[1]};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int v = 4 * g4 + e;
                        float p = s[v];  // exp2((S - lse / scale) * scale * log2 e) by now
                        if (MASKED) {
                            bool ok = (t0 + (unsigned)(8 * g4 + e) <= span) & some;
                            if (HAS_DOC) ok = ok & (ids[e] == dock);
                            p = ok ? p : 0.f;
                        }
                        const float ds = p * dp[v];
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
                    *(MA_GLB u32x4*)(ds_out + ds_lane + 64 * mb + 32 * pr) = u32x4{s0[0], s1[0], s0[1], s1[1]};
                }
            }
            // dV^T += dO^T P and dK^T += Q^T dS  (accumulators stay in AGPRs)
            // (one read pipeline for both products: it is filled once, and one fence serves both)
            MA_TICK(4);
            trfrag_gemm_two<D, 2, kBPipe>(lds_addr(Gs) + tbase + roff, pf, dvacc, lds_addr(Qs) + tbase + roff, dsf, dkacc, b_hook);
            MA_TICK(5);
        };
        block(std::integral_constant<int, 0>{});
        block(std::integral_constant<int, 1>{});
        MA_TICK(6);
        decode(nflags);
        ds_at = nds_at;
        have = have_next;
    }

    wait_vmem();      // (the chains of the last step have written to the free half of the ring: no test in the hooks)
    __syncthreads();  // everyone is done with the tiles: reuse the ring as store scratch
    mfma_fence();
    {
        constexpr int kPitchO = D * 2 + 16;
        const lds_ptr scratch = lds0 + w * 32 * kPitchO;
        __bf16* okp = (__bf16*)a.dk.ptr + b * a.dk.stride_b + hk * a.dk.stride_h;
        __bf16* ovp = (__bf16*)a.dv.ptr + b * a.dv.stride_b + hk * a.dv.stride_h;
        store_tile_T<D>(scratch, dkacc, a.scale, okp, a.dk.stride_s, kw_lo, S, lane);
        store_tile_T<D>(scratch, dvacc, 1.0f, ovp, a.dv.stride_s, kw_lo, S, lane);
    }
}

// One workgroup per work item, or -- with work queues in the tile map -- one per compute unit, pulling
// items until none is left (see WorkQueue).
template <int D, bool HAS_DOC, bool WRITE_DS, bool FULL>
__global__ __launch_bounds__(kBwdThreads, 1) void attn_bwd_dkv_bf16_kernel(AttnArgs a) {
    extern __shared__ __align__(16) char smem_raw[];
    MA_LDS int* box = (MA_LDS int*)((lds_ptr)smem_raw + (4 * Tile<D>::bytes(kStep) + 2 * kStep * (4 + 4 + 8)));
    WorkQueue wq;
    wq.init(a.map.work_counters, kQueueDkv, work_grid(a.B * a.T, a.Hkv, 1));
#ifdef MA_TICKS
    Ticks ticks;
    const unsigned long long t_start = __builtin_readcyclecounter();
    for (int id = wq.next(box); id >= 0; id = wq.next(box)) {
        MA_TICK(7);
        attn_bwd_dkv_bf16_item<D, HAS_DOC, WRITE_DS, FULL>(fresh_args(), id, ticks);
        __syncthreads();
        MA_TICK(8);
    }
    if (threadIdx.x == MA_T_WAVE * 64) {
        atomicAdd(&ma_dbg_ticks[0], ticks.acc);
        atomicAdd(&ma_dbg_ticks[1], (unsigned long long)ticks.n);
        atomicAdd(&ma_dbg_ticks[2], __builtin_readcyclecounter() - t_start);
        atomicAdd(&ma_dbg_ticks[3], 1ull);
    }
#else
    for (int id = wq.next(box); id >= 0; id = wq.next(box)) {
        attn_bwd_dkv_bf16_item<D, HAS_DOC, WRITE_DS, FULL>(fresh_args(), id);
        __syncthreads();  // the item's LDS (and the box) are free again
    }
#endif
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
    StepTable<BN> st;
    {
        int lo, hi;
        visibility_limits(false, i * kTile, i * kTile + kTile - 1, BN, bounded, wlim, windowed, lo, hi);
        int n_partial, n_full;
        // (the id range of the wave's own rows comes in the same round trip as the list lengths)
        if (use_rng) scalar_load2_range(a.map.kv_num_blocks + mrow, a.map.full_kv_num_blocks + mrow,
                                        rng_row + (size_t)(min(qw_lo, a.S - 1) / MA_DOC_BLOCK) * 2, n_partial, n_full, own);
        else scalar_load2(a.map.kv_num_blocks + mrow, a.map.full_kv_num_blocks + mrow, n_partial, n_full);
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
// dS^T is read exactly once, by the workgroup that owns its q tile: its loads carry the non-temporal hint, so that
// they do not displace the K tiles that the workgroups of a document share (dQ -2.5 % on the Gemma-3-4B shape)
constexpr bool kDsReadOnce = true;
constexpr int kDqPairMinD = 64;   // head dims from which an even GQA group goes through the two-head kernel
// dQ^T += K^T dS^T and nothing else: no Q / dO / O fragments, no scores, no exponentials.  Per step
// of 64 kv rows the workgroup stages the K tile and the [64 kv][128 q] slab of dS^T of its q tile;
// both MFMA operands come from LDS through transposed reads of the same kv rows, so their
// contraction orders agree by construction.  Every 32 x 32 block this kernel multiplies has been written: the
// dK/dV kernel walks the transposed tile lists and skips a block by the same tests as this kernel does (see
// WRITE_DS there); the slabs are staged whole, and what lies in the blocks nobody wrote is never used.
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
    StepTable<BN, true> st;
    st.numbering(a.map.tile_slot, ((int64_t)b * a.T + i) * a.T, 1, a.ds_tiles);     // tile (i, j) of this batch row, j walked
    {
        int lo, hi;
        visibility_limits(false, i * kTile, i * kTile + kTile - 1, BN, bounded, wlim, windowed, lo, hi);
        int n_partial, n_full;
        // (the id range of the wave's own rows comes in the same round trip as the list lengths)
        if (use_rng) scalar_load2_range(a.map.kv_num_blocks + mrow, a.map.full_kv_num_blocks + mrow,
                                        rng_row + (size_t)(min(qw_lo, a.S - 1) / MA_DOC_BLOCK) * 2, n_partial, n_full, own);
        else scalar_load2(a.map.kv_num_blocks + mrow, a.map.full_kv_num_blocks + mrow, n_partial, n_full);
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
        ss.template issue<kDsReadOnce>(sp + (size_t)(uint32_t)st.tile_slot * (kTile * kTile) + (size_t)(st.r0 & (kTile - 1)) * kTile, Sbuf(buf), w, lane, BN, kTile);   // the step's 64 kv rows inside its tile's slot
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
    StepTable<BN, true> st;
    st.numbering(a.map.tile_slot, ((int64_t)b * a.T + i) * a.T, 1, a.ds_tiles);     // tile (i, j) of this batch row, j walked
    {
        int lo, hi;
        visibility_limits(false, i * kTile, i * kTile + kTile - 1, BN, bounded, wlim, windowed, lo, hi);
        int n_partial, n_full;
        // (the id range of the wave's own rows comes in the same round trip as the list lengths)
        if (use_rng) scalar_load2_range(a.map.kv_num_blocks + mrow, a.map.full_kv_num_blocks + mrow,
                                        rng_row + (size_t)(min(qw_lo, a.S - 1) / MA_DOC_BLOCK) * 2, n_partial, n_full, own);
        else scalar_load2(a.map.kv_num_blocks + mrow, a.map.full_kv_num_blocks + mrow, n_partial, n_full);
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
        ss.template issue<kDsReadOnce>(sp0 + at, Sbuf(buf, 0), w, lane, BN, kTile);
        ss.template issue<kDsReadOnce>(sp1 + at, Sbuf(buf, 1), w, lane, BN, kTile);
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
                        ss.template issue_one<run, kDsReadOnce>(s0src, s0dst, w, s_lim, kTile * 2);
                    } else {
                        ss.template issue_one<run - decltype(ss)::PER, kDsReadOnce>(s1src, s1dst, w, s_lim, kTile * 2);
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

// FULL: every q step of the sequence has all of its rows (see the kernel's run_to_lds)
template <int D, bool HAS_DOC, bool WRITE_DS, bool FULL>
static int launch_dkv(const AttnArgs& a, size_t lds_kv, hipStream_t st) {
    int rc = opt_in_lds(attn_bwd_dkv_bf16_kernel<D, HAS_DOC, WRITE_DS, FULL>, lds_kv, "attn_bwd_dkv_bf16");
    if (rc) return rc;
    static const int resident = resident_workgroups(attn_bwd_dkv_bf16_kernel<D, HAS_DOC, WRITE_DS, FULL>, kBwdThreads, lds_kv);
    hipLaunchKernelGGL((attn_bwd_dkv_bf16_kernel<D, HAS_DOC, WRITE_DS, FULL>), dim3(queue_grid(work_grid(a.B * a.T, a.Hkv, 1), a.map.work_counters, resident), 1, 1),
                       dim3(kBwdThreads), lds_kv, st, a);
    return check_launch("attn_bwd_dkv_bf16_kernel");
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
        hipLaunchKernelGGL(attn_delta_bf16_kernel<D>, dim3((unsigned)((nrows + RPB * kDeltaRows - 1) / (RPB * kDeltaRows))), dim3(256), 0, st, a);
        rc = check_launch("attn_delta_bf16_kernel");
        if (rc) return rc;
    }
    const size_t lds_kv = (size_t)4 * Tile<D>::bytes(kStep) + 2 * kStep * (4 + 4 + 8) + 16 + (kBwdThreads / 64) * kDkvRecBytes;  // + work-queue box, step records
    if (hand_over) {
        if (a.stages & MA_BWD_DKV) {
            rc = a.S % kStep == 0 ? launch_dkv<D, HAS_DOC, true, true>(a, lds_kv, st) : launch_dkv<D, HAS_DOC, true, false>(a, lds_kv, st);
            if (rc) return rc;
        }
        const int G = a.Hq / a.Hkv;
        if ((a.stages & MA_BWD_DQ) && G % 2 == 0 && D >= kDqPairMinD) {
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
        rc = a.S % kStep == 0 ? launch_dkv<D, HAS_DOC, false, true>(a, lds_kv, st) : launch_dkv<D, HAS_DOC, false, false>(a, lds_kv, st);
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

#ifdef MA_TICKS
extern "C" void ma_dbg_read_ticks(unsigned long long* out, int reset) {
    (void)hipMemcpyFromSymbol(out, HIP_SYMBOL(ma::ma_dbg_ticks), sizeof(unsigned long long) * 4);
    if (reset) { unsigned long long z[4] = {0, 0, 0, 0}; (void)hipMemcpyToSymbol(HIP_SYMBOL(ma::ma_dbg_ticks), z, sizeof(z)); }
}
#endif
