// GQA flash-style forward for bf16 activations, two query heads per workgroup.
//
// Same contract as attn_fwd_bf16_kernel (maester/models/gemma/model.py:384-396; semantics
// torch/_higher_order_ops/flex_attention.py:159-267), for head layouts where an even number of
// query heads shares each kv head (enable_gqa, model.py:395).  A workgroup owns a 128-row q tile of
// TWO query heads of one kv head; wave w owns rows 32w..32w+31 of both.  The two heads read the
// same K and V, have the same mask and walk the same kv list, so per kv step the workgroup
//   * stages K/V once (half the global -> LDS traffic per FLOP),
//   * reads every K row fragment and every transposed V fragment from LDS once and feeds it to two
//     MFMAs (half the LDS reads per MFMA: the transposed reads bound the single-head kernel),
//   * evaluates the mask once,
// and the per-step control, the barrier and the per-workgroup prologue/epilogue are paid once for
// twice the work.  The price is registers: both O^T accumulators fill all 256 AGPRs, both heads' Q
// fragments take 128 VGPRs, so the 64-row kv step is consumed as two 32-row blocks.
//
// With the accumulators in AGPRs and no register to spare, there is no cheap way to multiply O^T by
// a per-row factor, so the online softmax never rescales: a row's reference maximum is set by its
// first visible block and exp2(score - reference) may grow up to 2^kSlack (exact in fp32 / bf16, a
// power-of-two scale).  If some row ever outgrows that, the workgroup notes it, finishes the walk,
// and redoes its tile in two passes: one that only finds the exact row maxima, one that accumulates
// against them.  That costs the workgroup half a forward more, and takes scores that span more than
// kSlack * ln 2 (44 nats) above a row's first block to happen.
#include "common.h"
#include "mfma.h"

namespace ma {

#ifdef MA_TICKS
// measurement builds only (maester_amd/kernel_ticks.py): cycles a wave spends between two of the marks
// MA_TICK(n) of the kernel; in the library the marks compile to nothing
__device__ unsigned long long ma_dbg_ticks_fwd[4];
struct TicksF {
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

constexpr int kPairThreads = 256;
constexpr int kPairBN = 64;   // kv rows staged per step
constexpr int kPairPipeK = 2;  // LDS fragment reads in flight ahead of the MFMAs (registers are tight)
constexpr int kPairPipeV = 2;
// Which chain of a step carries which of the next step's tile loads, in eighths of a wave's runs:
// kPairPlan[block][chain (0: S^T, 1: O^T)] = {tile (0: K, 1: V), first eighth, eighths}.  K rides in S^T
// chains only (the pass that only finds row maxima has no O^T chains, and needs no V).
// (K in the first block's S^T chain, V in the second block's: V in an O^T chain measured slower.)
constexpr int kPairPlan[2][2][3] = {{{0, 0, 8}, {0, 0, 0}}, {{1, 0, 8}, {0, 0, 0}}};

// The kv steps of one work item, resolved ahead of the loop that runs them.  A wave that has its SIMD to
// itself pays four cycles for every instruction it issues between two MFMA chains, so whatever a step
// needs is worked out 64 steps at a time, one candidate step per lane, and kept as a record of
// ready-made addresses in the wave's own slice of LDS; taking a step is then two broadcast LDS reads
// and a few v_readfirstlane.
//   word 0       first kv row | act1 << 29 | act0 << 30 | partial << 31
//   word 1       rows of the step that lie inside the sequence (1 .. 64)
//                (act0 / act1: this wave has something to do in the first / second 32-row block)
//   words 2,3    address of the step's first K row        words 4,5    of its first V row
//   words 6,7    of the document id of its first row (HAS_DOC)
// Every wave of a workgroup derives the same sequence of steps (same inputs); only the two block bits
// are its own.  Nothing a refill needs is kept between refills except the position in the walk: it is
// derived again from the argument block, so that the step loop holds no registers for it.
constexpr int kPairRecWords = 8;
constexpr int kPairRecBytes = 64 * kPairRecWords * 4;  // LDS per wave
template <bool HAS_DOC>
struct PairSteps {
    MA_LDS uint32_t* tab;
    int cbase, cnt, pos;
    __device__ __forceinline__ void start(MA_LDS uint32_t* table) { tab = table; cbase = 0; cnt = 0; pos = -1; }

    // the next candidates that hold a step at all; false when the walk is over.
    // FIRST (an item's first fill): the candidates are scanned at least once, and `mid1` / `mid2` run
    // while the scan's two dependent loads (list entries, then id ranges of the blocks) are on their way
    // -- the item's own operand loads go there, so that the round trips do not queue up behind them.
    // Every load of the scan is unconditional (a load under a condition is waited for on the spot).
    template <bool FIRST, class F1, class F2>
    __device__ __forceinline__ bool refill(const int i, const int hk, const int b, const int w, F1&& mid1, F2&& mid2) {
        KernArgs& a = fresh_args();
        const int lane = __lane_id();
        const size_t mrow = (size_t)b * a.T + i;
        const bool use_rng = HAS_DOC && a.map.block_doc_range != nullptr;
        const int64_t* rng = use_rng ? a.map.block_doc_range + (size_t)b * (2 * ((a.S + 63) / 64)) * 2 : nullptr;
        const int qw_lo = i * kTile + 32 * w, qw_hi = qw_lo + 31;
        DocRange own;  // id range of the wave's own q rows: in the same round trip as the list lengths
        int np, nf;
        if (use_rng) scalar_load2_range(a.map.kv_num_blocks + mrow, a.map.full_kv_num_blocks + mrow,
                                        rng + (size_t)(min(qw_lo, a.S - 1) / MA_DOC_BLOCK) * 2, np, nf, own);
        else scalar_load2(a.map.kv_num_blocks + mrow, a.map.full_kv_num_blocks + mrow, np, nf);
        const int n = np + nf, total = n * (kTile / kPairBN);
        const bool bounded = a.causal || a.window >= 0, windowed = a.window >= 0;
        const int wlim = windowed ? (int)min(a.window, (int64_t)0x3fffffff) : 0x7fffffff;
        int vis_lo, vis_hi, blk_lo, blk_hi;
        visibility_limits(false, i * kTile, i * kTile + kTile - 1, kPairBN, bounded, wlim, windowed, vis_lo, vis_hi);
        visibility_limits(false, qw_lo, qw_hi, 32, bounded, wlim, windowed, blk_lo, blk_hi);
        int64_t own_lo = 0, own_hi = 0;
        if (use_rng) {
            own_lo = own.lo();
            own_hi = own.hi();
        }
        const int32_t* pl = a.map.kv_indices + mrow * a.T;
        const int32_t* fl = a.map.full_kv_indices + mrow * a.T;
        const char* kp = (const char*)((const __bf16*)a.k.ptr + b * a.k.stride_b + hk * a.k.stride_h);
        const char* vp = (const char*)((const __bf16*)a.v.ptr + b * a.v.stride_b + hk * a.v.stride_h);
        const uint32_t ksb = (uint32_t)(a.k.stride_s * 2), vsb = (uint32_t)(a.v.stride_s * 2);
        cnt = 0;
        auto scan = [&](auto first_c) {
            constexpr bool first = decltype(first_c)::value;
            const int c = cbase + lane;
            const bool valid = c < total;
            const int cc = valid ? c : 0;
            const int idx = cc / (kTile / kPairBN), half = cc - idx * (kTile / kPairBN);
            const bool partial = idx < np;
            const int32_t* entry = partial ? pl + idx : fl + (idx - np);  // (no candidate: the first entry of a list, unused)
            int tile = *(const MA_GLB int32_t*)entry;
            if constexpr (first) {
                asm volatile("" ::: "memory");
                mid1();
                asm volatile("" ::: "memory");
            }
            tile = valid ? tile : 0;
            const int r0 = tile * kTile + half * kPairBN;
            const bool vis = valid & (r0 < a.S) & (!partial | ((r0 >= vis_lo) & (r0 <= vis_hi)));
            bool act0 = (r0 < a.S) & (!partial | ((r0 >= blk_lo) & (r0 <= blk_hi)));
            bool act1 = (r0 + 32 < a.S) & (!partial | ((r0 + 32 >= blk_lo) & (r0 + 32 <= blk_hi)));
            if constexpr (HAS_DOC) {
                // id ranges of the step's two blocks; where there is nothing to look up (no range table, a full
                // tile, no step) the load reads the head of the K tensor instead and its result is not used
                const bool look = use_rng & partial & vis;
                const MA_GLB i64x2* e = (const MA_GLB i64x2*)(look ? (const void*)(rng + (size_t)(r0 / 32) * 2) : (const void*)kp);
                const i64x2 e0 = e[0], e1 = e[1];
                if constexpr (first) {
                    asm volatile("" ::: "memory");
                    mid2();
                    asm volatile("" ::: "memory");
                }
                // no row of the block shares a document with the wave's own rows
                act0 &= !look | ((e0[0] <= own_hi) & (e0[1] >= own_lo));
                act1 &= !look | ((e1[0] <= own_hi) & (e1[1] >= own_lo));
            } else if constexpr (first) {
                mid2();
            }
            const uint64_t mask = __ballot(vis);
            const int at = __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
            if (vis) {
                const uint64_t ka = (uint64_t)(kp + (uint64_t)(uint32_t)r0 * ksb), va = (uint64_t)(vp + (uint64_t)(uint32_t)r0 * vsb);
                const uint64_t da = HAS_DOC ? (uint64_t)(a.doc + (size_t)b * a.S + r0) : 0;
                MA_LDS uint32_t* rec = tab + at * kPairRecWords;
                *(MA_LDS u32x4*)rec = u32x4{(uint32_t)r0 | ((uint32_t)act1 << 29) | ((uint32_t)act0 << 30) | ((uint32_t)partial << 31),
                                            (uint32_t)min(kPairBN, a.S - r0), (uint32_t)ka, (uint32_t)(ka >> 32)};
                *(MA_LDS u32x4*)(rec + 4) = u32x4{(uint32_t)va, (uint32_t)(va >> 32), (uint32_t)da, (uint32_t)(da >> 32)};
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
    __device__ __forceinline__ bool advance(const int i, const int hk, const int b, const int w) {
        if (++pos < cnt) return true;
        return refill<false>(i, hk, b, w, [] {}, [] {});
    }
    // the first step of an item (call after start())
    template <class F1, class F2>
    __device__ __forceinline__ bool advance_first(const int i, const int hk, const int b, const int w, F1&& mid1, F2&& mid2) {
        return refill<true>(i, hk, b, w, mid1, mid2);
    }
};
__device__ __forceinline__ uint64_t pair_uniform64(uint32_t lo, uint32_t hi) {
    return (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane(lo) | ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane(hi) << 32);
}

template <int D, bool HAS_DOC, bool FULL>
__device__ __forceinline__ void attn_fwd_pair_bf16_item(KernArgs& a, const int wg_id
#ifdef MA_TICKS
    , TicksF& ticks
#endif
) {
    using TL = Tile<D>;
    constexpr int KK = D / 16;
    constexpr int DB = D / 32;
    constexpr int BN = kPairBN;
    constexpr int NW = kPairThreads / 64;
    extern __shared__ __align__(16) char smem_raw[];
    const lds_ptr lds0 = (lds_ptr)smem_raw;
    auto Kbuf = [&](int i) { return lds0 + i * 2 * TL::bytes(BN); };
    auto Vbuf = [&](int i) { return lds0 + i * 2 * TL::bytes(BN) + TL::bytes(BN); };
    auto Dbuf = [&](int i) { return (MA_LDS int64_t*)(lds0 + 4 * TL::bytes(BN)) + i * BN; };

    const int tid = fresh_tid(), lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, hh = lane >> 5;
    const int G = a.Hq / a.Hkv, GP = G / 2;  // head pairs per kv head
    int i, hp, b;
    if (!map_work(wg_id, a.B * a.T, a.T, a.Hkv, GP, a.map.q_tile_order, i, hp, b)) return;
    MA_TICK(9);
    const int hk = hp / GP;
    const int h0 = hk * G + 2 * (hp % GP);   // the pair is (h0, h0 + 1)
    const int qw_lo = i * kTile + 32 * w;
    const int q = qw_lo + r;
    const bool qvalid = q < a.S;
    const bool bounded = a.causal || a.window >= 0;

    const __bf16* qp = (const __bf16*)a.q.ptr + b * a.q.stride_b + h0 * a.q.stride_h;
    const uint32_t ksb = (uint32_t)(a.k.stride_s * 2), vsb = (uint32_t)(a.v.stride_s * 2);
    const int64_t* drow = HAS_DOC ? a.doc + (size_t)b * a.S : nullptr;
    const int rbase = TL::row_base(lane), tbase = TL::tr_base(lane);

    const int qc = min(q, a.S - 1);
    const int64_t docq = HAS_DOC ? drow[qc] : 0;
    const bool windowed = a.window >= 0;
    const int wlim = windowed ? (int)min(a.window, (int64_t)0x3fffffff) : 0x7fffffff;
    const float sl2 = a.scale * kLog2e;

    // The K and V tiles have the same shape: one set of slots.  Every wave moves the same number of runs
    // of a tile from inside its MFMA chains (kPaced); the run that is left over (a tile is 4 * kPaced + 1
    // runs) is moved by wave 0 (K) or wave 1 (V) when the step begins.
    using SK = DirectStager<D, BN, NW>;
    constexpr int kPaced = (SK::NL - 1) / NW;
    static_assert(SK::NL == NW * kPaced + 1 && (2 * KK) % kPaced == 0 && 4 * DB == 2 * KK, "tile runs per wave");
    // the lane's byte offset into a K tile and into a V tile for each of its runs (the two tensors may have
    // different row strides), and for the left-over run of the tile its wave moves
    uint32_t koff[kPaced], voff[kPaced], off_last;
    {
        int row, chunk;
#pragma unroll
        for (int p = 0; p < kPaced; ++p) {
            SK::slot(w + p * NW, lane, row, chunk);
            koff[p] = (uint32_t)row * ksb + (uint32_t)chunk * 16u;
            voff[p] = (uint32_t)row * vsb + (uint32_t)chunk * 16u;
        }
        SK::slot(SK::NL - 1, lane, row, chunk);
        off_last = (uint32_t)row * (w == 0 ? ksb : vsb) + (uint32_t)chunk * 16u;
    }
    constexpr uint32_t kRowBytes = D * 2;
    // Where a run comes from.  FULL (the sequence is a whole number of tiles, so every tile has all of its
    // rows): the tile's address, and a run is a plain load into LDS -- on the last step of a walk, when there
    // is no next tile, the address stays on the current one, which is read once more.  Otherwise: a buffer
    // descriptor of the tile with `rows` rows in range; lanes of rows past it (all of them when there is no
    // next tile) read nothing and zeros land in LDS.  (The plain load is the faster instruction here.)
    struct Src { uint64_t at; u32x4 rsrc; };
    auto k_tile = [&](uint64_t at, int rows) {
        Src t{at, u32x4{0, 0, 0, 0}};
        if constexpr (!FULL) t.rsrc = tile_rsrc(at, rows > 0 ? (uint32_t)(rows - 1) * ksb + kRowBytes : 0u);
        return t;
    };
    auto v_tile = [&](uint64_t at, int rows) {
        Src t{at, u32x4{0, 0, 0, 0}};
        if constexpr (!FULL) t.rsrc = tile_rsrc(at, rows > 0 ? (uint32_t)(rows - 1) * vsb + kRowBytes : 0u);
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
    int64_t kd_next = 0;

    // The walk over the kv tiles: its index loads go out first, then both heads' Q rows, which go
    // straight from global memory into MFMA operand fragments (lane (r, hh): elements 16*kk + 8*hh
    // .. +7 of row qw_lo + r, one 16-byte load each; nothing passes through LDS), then, once the
    // index loads are back, the first K/V tiles -- all in flight together.
    // (the fields of the current step's word are carried as variables of their own: decoded from the word
    // inside the loop, the compiler splits the accumulators' live ranges around the skipped-block path
    // and spills them)
    bool have;
    int k0 = 0;
    bool partial = false, act0 = false, act1 = false;  // of the step the walk stands on: tile kind, blocks this wave has work in
    uint64_t k_at = 0, v_at = 0;                       // its K and V rows
    auto decode = [&](uint32_t word) {
        k0 = (int)(word & 0xffffffu);
        partial = (word >> 31) != 0;
        act0 = (word >> 30) & 1u;
        act1 = (word >> 29) & 1u;
    };
    PairSteps<HAS_DOC> st;
    // document ids of a partial step's kv rows: every wave loads them for the step after the current
    // one (no branch: a conditional load would be waited for on the spot), wave 3 writes them to LDS
    auto load_ids = [&](uint64_t doc_at, int rows) {
        if (HAS_DOC) kd_next = ((const MA_GLB int64_t*)doc_at)[min(lane, rows - 1)];
    };
    // O^T of both heads: all 256 AGPRs (D = 256); nothing but MFMAs touches them inside the loop
    f32x16 oa[DB], ob[DB];
    auto zero_acc = [&]() {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) oa[db][v] = ob[db][v] = 0.f;
        pin_tiles<0, DB, true>(oa);
        pin_tiles<0, DB, true>(ob);
    };
    bf16x8 qa[KK], qb[KK];
    const __bf16* qrow = qp + (int64_t)qc * a.q.stride_s + 8 * hh;
    auto load_qa = [&]() {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) qa[kk] = *(const bf16x8*)(qrow + 16 * kk);
    };
    auto load_qb = [&]() {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) qb[kk] = *(const bf16x8*)(qrow + a.q.stride_h + 16 * kk);
        zero_acc();  // (while the loads are on their way)
    };
    auto walk_first = [&](auto first_c) {
        st.start((MA_LDS uint32_t*)(lds0 + 4 * TL::bytes(BN) + 2 * BN * 8 + 16) + w * (kPairRecBytes / 4));
        if constexpr (decltype(first_c)::value) have = st.advance_first(i, hk, b, w, load_qa, load_qb);
        else have = st.advance(i, hk, b, w);
        MA_TICK(17);
        if (have) {
            MA_LDS uint32_t* rec = st.tab + st.pos * kPairRecWords;
            const u32x4 x0 = *(MA_LDS u32x4*)rec, x1 = *(MA_LDS u32x4*)(rec + 4);
            decode(__builtin_amdgcn_readfirstlane(x0[0]));
            k_at = pair_uniform64(x0[2], x0[3]);
            v_at = pair_uniform64(x1[0], x1[1]);
            const int rows_valid = (int)__builtin_amdgcn_readfirstlane(x0[1]);
            const Src kr = k_tile(k_at, rows_valid), vr = v_tile(v_at, rows_valid);
#pragma unroll
            for (int p = 0; p < kPaced; ++p) run_to_lds(kr, koff[p], lds_addr(Kbuf(0)) + (w + p * NW) * 1024);
            if (w == 0) run_to_lds(kr, off_last, lds_addr(Kbuf(0)) + (SK::NL - 1) * 1024);
#pragma unroll
            for (int p = 0; p < kPaced; ++p) run_to_lds(vr, voff[p], lds_addr(Vbuf(0)) + (w + p * NW) * 1024);
            if (w == 1) run_to_lds(vr, off_last, lds_addr(Vbuf(0)) + (SK::NL - 1) * 1024);
            load_ids(pair_uniform64(x1[2], x1[3]), rows_valid);
        }
    };
    MA_TICK(16);
    walk_first(std::true_type{});
    MA_TICK(10);
    float ma_ = -INFINITY, mb_ = -INFINITY, la = 0.f, lb = 0.f;
    MA_LDS int* outgrown = (MA_LDS int*)(lds0 + 4 * TL::bytes(BN) + 2 * BN * 8);
    if (tid == 0) *outgrown = 0;
    constexpr float kSlack = 32.0f;

    // mode 0: the one pass described above; mode 1: row maxima only; mode 2: accumulate against them
    for (int mode = 0;; ) {
    la = lb = 0.f;
    if (mode != 2) ma_ = mb_ = -INFINITY;
    if (mode) {  // a later pass starts the walk again (the first pass cleared the accumulators while its loads were on their way)
        zero_acc();
        walk_first(std::false_type{});
    }
    MA_TICK(11);

    for (int n = 0; have; ++n) {
        MA_TICK(0);
        const int cur = n & 1;
        const lds_ptr Ks = Kbuf(cur), Vs = Vbuf(cur);
        MA_LDS int64_t* kdoc = Dbuf(cur);
        if (HAS_DOC && w == 3) kdoc[lane] = kd_next;
        const bool have_next = st.advance(i, hk, b, w);
        u32x4 x0 = {0, 0, 0, 0}, x1 = x0;
        if (have_next) {  // the record of the next step: read now, picked up behind the barrier
            MA_LDS uint32_t* rec = st.tab + st.pos * kPairRecWords;
            x0 = *(MA_LDS u32x4*)rec;
            x1 = *(MA_LDS u32x4*)(rec + 4);
        }
        wait_vmem();
        MA_TICK(20);
        __syncthreads();
        MA_TICK(1);

        const int ck0 = k0;
        const bool cpartial = partial;
        const bool act[2] = {act0, act1};
        uint32_t nword = 0;
        // The tile loads of the next step ride in this step's chains, one run every few MFMAs (see
        // kPairPlan): issued in one burst they fill the memory pipeline and stall the wave with the
        // matrix cores idle.  On the last step of a walk the loads stay in the chains -- cheaper than a test
        // in every hook -- and fill the free half of the ring with the current tiles once more, or with zeros
        // (see run_to_lds).
        int nrows = 0;
        if (have_next) {
            nword = __builtin_amdgcn_readfirstlane(x0[0]);
            k_at = pair_uniform64(x0[2], x0[3]);
            v_at = pair_uniform64(x1[0], x1[1]);
            nrows = (int)__builtin_amdgcn_readfirstlane(x0[1]);  // (from the record: the sequence length is not kept in a register)
            load_ids(pair_uniform64(x1[2], x1[3]), nrows);
        }
        const Src kr = k_tile(k_at, nrows), vr = v_tile(v_at, nrows);
        if (have_next) {
            if (w == 0) run_to_lds(kr, off_last, lds_addr(Kbuf(cur ^ 1)) + (SK::NL - 1) * 1024);
            if (w == 1 && mode != 1) run_to_lds(vr, off_last, lds_addr(Vbuf(cur ^ 1)) + (SK::NL - 1) * 1024);
        }
        const uint32_t kdst = lds_addr(Kbuf(cur ^ 1)) + w * 1024, vdst = lds_addr(Vbuf(cur ^ 1)) + w * 1024;  // the wave's first run

        // mask constants of this step (see attn_fwd_bf16_kernel)
        const int qrel = q - ck0 - 4 * hh;
        const int dlo = max(bounded ? 0 : -0x40000000, q - a.S + 1);
        const unsigned span = (unsigned)(wlim - dlo);
        const bool some = wlim >= dlo;
        const unsigned t0 = (unsigned)(qrel - dlo);

        // The two 32-row blocks of the step are two copies of the same code (nb is a compile-time
        // constant in each), so that each chain carries exactly the loads planned for it.
        auto block = [&](auto nb_c) {
            constexpr int nb = decltype(nb_c)::value;
            MA_TICK(2);
            constexpr int kPlanA[3] = {kPairPlan[nb][0][0], kPairPlan[nb][0][1] * kPaced / 8, kPairPlan[nb][0][2] * kPaced / 8};
            constexpr int kPlanB[3] = {kPairPlan[nb][1][0], kPairPlan[nb][1][1] * kPaced / 8, kPairPlan[nb][1][2] * kPaced / 8};
            static_assert(kPlanB[2] == 0 || kPlanB[0] == 1, "K rides in S^T chains only");
            auto move_run = [&](auto tile_c, auto run_c) {
                constexpr int run = decltype(run_c)::value;
                if constexpr (decltype(tile_c)::value == 0)
                    run_to_lds_at(kr, koff[run], kdst, std::integral_constant<int, run * (NW * 1024)>{});
                else
                    run_to_lds_at(vr, voff[run], vdst, std::integral_constant<int, run * (NW * 1024)>{});
            };
            auto burst_plan = [&](auto plan_c) {
                constexpr int which = decltype(plan_c)::value;
                constexpr int tile = which ? kPlanB[0] : kPlanA[0], first = which ? kPlanB[1] : kPlanA[1], count = which ? kPlanB[2] : kPlanA[2];
                static_for<0, count>([&](auto r) { move_run(std::integral_constant<int, tile>{}, std::integral_constant<int, first + decltype(r)::value>{}); });
            };
            if (!act[nb]) {
                if (have_next) {  // the loads its chains would have carried
                    burst_plan(std::integral_constant<int, 0>{});
                    if (mode != 1) burst_plan(std::integral_constant<int, 1>{});
                }
                return;
            }
            auto a_hook = [&](auto idx) {
                constexpr int c = decltype(idx)::value;
                if constexpr (kPlanA[2] > 0) {
                    constexpr int every = (2 * KK) / kPlanA[2];
                    if constexpr (c % every == every - 1) move_run(std::integral_constant<int, kPlanA[0]>{}, std::integral_constant<int, kPlanA[1] + c / every>{});
                }
            };
            auto b_hook = [&](auto idx) {
                constexpr int c = decltype(idx)::value;
                if constexpr (kPlanB[2] > 0) {
                    constexpr int every = (2 * KK) / kPlanB[2];
                    if constexpr (c % every == every - 1) move_run(std::integral_constant<int, kPlanB[0]>{}, std::integral_constant<int, kPlanB[1] + c / every>{});
                }
            };
            const uint32_t roff = (uint32_t)(32 * nb * TL::kPitch);

            // S^T of both heads for 32 kv rows (lane owns one q row, 16 of the kv rows)
            f32x16 sa, sb;
            rowfrag_gemm_dual<D, kPairPipeK>(lds_addr(Ks) + rbase + roff, qa, qb, sa, sb, a_hook);
            MA_TICK(3);

            // mask (shared by the two heads)
            if (cpartial) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    i64x2 id01 = {0, 0}, id23 = {0, 0};
                    if (HAS_DOC) {
                        id01 = *(MA_LDS i64x2*)(kdoc + 32 * nb + 8 * g + 4 * hh);
                        id23 = *(MA_LDS i64x2*)(kdoc + 32 * nb + 8 * g + 4 * hh + 2);
                    }
                    const int64_t ids[4] = {id01[0], id01[1], id23[0], id23[1]};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int v = 4 * g + e;
                        bool ok = (t0 - (unsigned)(32 * nb + 8 * g + e) <= span) & some;
                        if (HAS_DOC) ok = ok & (ids[e] == docq);
                        sa[v] = ok ? sa[v] : -INFINITY;
                        sb[v] = ok ? sb[v] : -INFINITY;
                    }
                }
            }
            // Once every row of the wave has its reference, a block needs no row maxima: the scores
            // are exponentiated against the references and a row that outgrows the slack shows in its
            // sum (a sum above 2^kSlack sends the workgroup into the redo, as a single term would).
            const bool settled = (mode != 1) & !__any((ma_ == -INFINITY) | (mb_ == -INFINITY));
            if (!settled) {
                float mxa = -INFINITY, mxb = -INFINITY;  // row maxima on the unscaled scores
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    mxa = fmaxf(mxa, sa[v]);
                    mxb = fmaxf(mxb, sb[v]);
                }
                mxa = fmaxf(mxa, xor32(mxa)) * sl2;   // the (positive) scale goes into the exponent's multiply-add
                mxb = fmaxf(mxb, xor32(mxb)) * sl2;
                if (mode == 1) {  // maxima only
                    ma_ = fmaxf(ma_, mxa);
                    mb_ = fmaxf(mb_, mxb);
                    return;
                }
                if (mode == 0) {
                    // the first visible block sets the reference; a later block that outgrows it by more
                    // than kSlack log2 units sends the workgroup into the two-pass redo
                    const bool late = ((ma_ != -INFINITY) & (mxa > ma_ + kSlack)) | ((mb_ != -INFINITY) & (mxb > mb_ + kSlack));
                    if (__any(late) && lane == 0) *outgrown = 1;
                    ma_ = ma_ == -INFINITY ? mxa : ma_;
                    mb_ = mb_ == -INFINITY ? mxb : mb_;
                }
            }
            const float mua = ma_ == -INFINITY ? 0.f : ma_, mub = mb_ == -INFINITY ? 0.f : mb_;
            float rsa = 0.f, rsb = 0.f;
            bf16x8 pa[2], pb[2];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float x = fast_exp2(__builtin_fmaf(sa[v], sl2, -mua));
                const float y = fast_exp2(__builtin_fmaf(sb[v], sl2, -mub));
                rsa += x;
                rsb += y;
                pa[v >> 3][v & 7] = (__bf16)x;
                pb[v >> 3][v & 7] = (__bf16)y;
            }
            if (settled && mode == 0) {
                constexpr float kTooLarge = 4294967296.0f;  // 2^kSlack
                static_assert(kSlack == 32.0f, "threshold of the row sums");
                if (__any((rsa > kTooLarge) | (rsb > kTooLarge)) && lane == 0) *outgrown = 1;
            }
            la += rsa;  // the lane's own 16 kv rows of the block; the two lanes of a q row are added at the end
            lb += rsb;

            // O^T += V^T P^T for both heads: every transposed V fragment feeds two MFMAs
            MA_TICK(4);
            trfrag_gemm_dual<D, 2, kPairPipeV>(lds_addr(Vs) + tbase + roff, pa, pb, oa, ob, b_hook);
            MA_TICK(5);
        };
        block(std::integral_constant<int, 0>{});
        block(std::integral_constant<int, 1>{});
        MA_TICK(6);
        if (have_next) decode(nword);
        have = have_next;
    }

    wait_vmem();      // (the chains of the last step have written to the free half of the ring)
    __syncthreads();  // every wave is done with the K/V buffers, and with the flag
    const int redo = *outgrown;
    if (mode == 0 && redo) { mode = 1; continue; }
    if (mode == 1) { mode = 2; continue; }
    break;
    }  // passes
    MA_TICK(12);

    // Epilogue: O^T (a lane owns one q row, 4 consecutive d per register group) goes through the
    // wave's LDS scratch so that the global stores are whole 16-byte-per-lane row segments.
    __syncthreads();  // every wave is done with the K/V buffers
    mfma_fence();
    MA_TICK(13);
    {
        constexpr int kPitchO = D * 2 + 16;
        lds_ptr Os = lds0 + w * 32 * kPitchO;
        constexpr int CH = D / 8, RPI = 64 / CH;
        const int rsub = lane / CH, c = lane % CH;
        const int64_t o_stride_s = a.o.stride_s;
        const uint32_t o_row_bytes = (uint32_t)(o_stride_s * 2);
        // (one copy of the code per head: picked at run time, every element would be read from both
        // accumulators and selected)
        static_for<0, 2>([&](auto hsel_c) {
            constexpr int hsel = decltype(hsel_c)::value;
            const float lp = hsel ? lb : la, m = hsel ? mb_ : ma_;
            const float l = lp + xor32(lp);
            const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    bf16x4 pk;
#pragma unroll
                    for (int e = 0; e < 4; ++e) pk[e] = (__bf16)((hsel ? ob[db][4 * g + e] : oa[db][4 * g + e]) * inv);
                    *(MA_LDS bf16x4*)(Os + r * kPitchO + (32 * db + 8 * g + 4 * hh) * 2) = pk;
                }
            }
            if constexpr (hsel == 0) MA_TICK(18);
            // all of the wave's rows leave LDS first, then go out: one LDS round trip and no dependent
            // scalar load per store (the row stride is read once, offsets are 32-bit)
            MA_GLB char* og = (MA_GLB char*)((__bf16*)a.o.ptr + b * a.o.stride_b + (h0 + hsel) * a.o.stride_h + (int64_t)qw_lo * o_stride_s);
            u32x4 val[32 / RPI];
#pragma unroll
            for (int it = 0; it < 32 / RPI; ++it) val[it] = *(MA_LDS u32x4*)(Os + (it * RPI + rsub) * kPitchO + c * 16);
            if constexpr (hsel == 0) MA_TICK(19);
            if (qw_lo + 31 < a.S) {
#pragma unroll
                for (int it = 0; it < 32 / RPI; ++it) *(MA_GLB u32x4*)(og + (uint32_t)(it * RPI + rsub) * o_row_bytes + c * 16) = val[it];
            } else {
#pragma unroll
                for (int it = 0; it < 32 / RPI; ++it)
                    if (qw_lo + it * RPI + rsub < a.S) *(MA_GLB u32x4*)(og + (uint32_t)(it * RPI + rsub) * o_row_bytes + c * 16) = val[it];
            }
            if (qvalid && hh == 0)
                a.lse[((size_t)b * a.Hq + h0 + hsel) * a.S + q] = l > 0.f ? (m + __log2f(l)) * kLn2 : -INFINITY;
            if constexpr (hsel == 0) { MA_TICK(14); } else { MA_TICK(15); }
        });
    }
}

// One workgroup per work item, or -- with work queues in the tile map -- one per compute unit, pulling
// items until none is left (see WorkQueue).
template <int D, bool HAS_DOC, bool FULL>
__global__ __launch_bounds__(kPairThreads) void attn_fwd_pair_bf16_kernel(AttnArgs a) {
    extern __shared__ __align__(16) char smem_raw[];
    MA_LDS int* box = (MA_LDS int*)((lds_ptr)smem_raw + (4 * Tile<D>::bytes(kPairBN) + 2 * kPairBN * 8 + 4));
    WorkQueue wq;
    wq.init(a.map.work_counters, kQueueFwd, work_grid(a.B * a.T, a.Hkv, a.Hq / a.Hkv / 2));
#ifdef MA_TICKS
    TicksF ticks;
    const unsigned long long t_start = __builtin_readcyclecounter();
    for (int id = wq.next(box); id >= 0; id = wq.next(box)) {
        MA_TICK(7);
        attn_fwd_pair_bf16_item<D, HAS_DOC, FULL>(fresh_args(), id, ticks);
        __syncthreads();
        MA_TICK(8);
    }
    if (threadIdx.x == MA_T_WAVE * 64) {
        atomicAdd(&ma_dbg_ticks_fwd[0], ticks.acc);
        atomicAdd(&ma_dbg_ticks_fwd[1], (unsigned long long)ticks.n);
        atomicAdd(&ma_dbg_ticks_fwd[2], __builtin_readcyclecounter() - t_start);
        atomicAdd(&ma_dbg_ticks_fwd[3], 1ull);
    }
#else
    for (int id = wq.next(box); id >= 0; id = wq.next(box)) {
        attn_fwd_pair_bf16_item<D, HAS_DOC, FULL>(fresh_args(), id);
        __syncthreads();  // the item's LDS (and the box) are free again
    }
#endif
    wq.leave();
}

template <int D, bool HAS_DOC, bool FULL>
static int pair_dd(const AttnArgs& a, hipStream_t st) {
    const size_t lds = (size_t)4 * Tile<D>::bytes(kPairBN) + 2 * kPairBN * 8 + 16 + (kPairThreads / 64) * kPairRecBytes;  // K/V ring, kv ids, redo flag + work-queue box, step records
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)attn_fwd_pair_bf16_kernel<D, HAS_DOC, FULL>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return fail(MA_ERR_LAUNCH, "hipFuncSetAttribute(attn_fwd_pair_bf16, %zu): %s", lds, hipGetErrorString(e));
    }
    const int GP = a.Hq / a.Hkv / 2;
    static const int resident = resident_workgroups(attn_fwd_pair_bf16_kernel<D, HAS_DOC, FULL>, kPairThreads, lds);
    hipLaunchKernelGGL((attn_fwd_pair_bf16_kernel<D, HAS_DOC, FULL>), dim3(queue_grid(work_grid(a.B * a.T, a.Hkv, GP), a.map.work_counters, resident), 1, 1),
                       dim3(kPairThreads), lds, st, a);
    return check_launch("attn_fwd_pair_bf16_kernel");
}

// Only for head layouts with an even number of query heads per kv head; the caller checks.
template <int D>
static int pair_d(const AttnArgs& a, hipStream_t st) {
    // every tile has all of its rows when the sequence is a whole number of kv steps
    const bool full = a.S % kPairBN == 0;
    if (a.doc) return full ? pair_dd<D, true, true>(a, st) : pair_dd<D, true, false>(a, st);
    return full ? pair_dd<D, false, true>(a, st) : pair_dd<D, false, false>(a, st);
}

int launch_attn_fwd_pair_bf16(const AttnArgs& a, hipStream_t st) {
    switch (a.D) {
        case 64: return pair_d<64>(a, st);
        case 128: return pair_d<128>(a, st);
        case 256: return pair_d<256>(a, st);
    }
    return fail(MA_ERR_UNSUPPORTED, "attn_fwd bf16: head_dim %d not in {64,128,256}", a.D);
}

}  // namespace ma

#ifdef MA_TICKS
extern "C" void ma_dbg_read_ticks_fwd(unsigned long long* out, int reset) {
    (void)hipMemcpyFromSymbol(out, HIP_SYMBOL(ma::ma_dbg_ticks_fwd), sizeof(unsigned long long) * 4);
    if (reset) { unsigned long long z[4] = {0, 0, 0, 0}; (void)hipMemcpyToSymbol(HIP_SYMBOL(ma::ma_dbg_ticks_fwd), z, sizeof(z)); }
}
#endif
