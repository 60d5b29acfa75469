// Shared declarations of the gfx950 packed-SFT attention library (internal; the public C ABI is
// include/maester_attn.h).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/maester_attn.h"

namespace ma {

// thread-local error message behind ma_last_error()
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);

constexpr int kTile = MA_TILE;  // BlockMask tile edge

// Mask predicate of maester/models/gemma/model.py:203-256 in device form.
struct MaskSpec {
    int causal;
    int64_t window;  // < 0: none
};

__device__ __forceinline__ bool pair_allowed(int q, int kv, int causal, int64_t window) {
    bool ok = true;
    if (causal) ok = ok && (q >= kv);
    if (window >= 0) ok = ok && (q >= kv) && ((int64_t)(q - kv) <= window);
    return ok;
}

// Launchers (each validates nothing: the C-ABI layer in api.hip has already done so).
int launch_tile_map(const int64_t* doc, int B, int S, int causal, int64_t window, const ma_tile_map& out,
                    void* ws, hipStream_t st);
// device address, on the current device, of the library-owned scratch behind ma_tile_map_build_static
int static_tile_map_scratch(void** out);
int launch_prologue_fwd(const ma_tensor4& qi, const ma_tensor4& ki, const ma_tensor4& qo, const ma_tensor4& ko,
                        const float* qw, const float* kw, const float* cs, const float* sn, int64_t n_pos,
                        const int64_t* pos, float eps, int unit, float* q_rstd, float* k_rstd, int dtype, int B,
                        int S, int Hq, int Hkv, int D, hipStream_t st);
int prologue_bwd_blocks(int B, int S);
int launch_prologue_bwd(const ma_tensor4& qi, const ma_tensor4& ki, const ma_tensor4& dqo, const ma_tensor4& dko,
                        const ma_tensor4& dqi, const ma_tensor4& dki, const float* qw, const float* kw,
                        const float* cs, const float* sn, int64_t n_pos, const int64_t* pos, int unit,
                        const float* q_rstd, const float* k_rstd, float* dqw, float* dkw, void* ws, int dtype,
                        int B, int S, int Hq, int Hkv, int D, hipStream_t st);

int launch_packed_ids(const int32_t* starts, const int32_t* lengths, const int32_t* counts, int B, int max_docs, int S,
                      int64_t* position_ids, int64_t* document_ids, hipStream_t st);

int rmsnorm_bwd_blocks(int64_t rows);
int launch_rmsnorm_fwd(const void* x, const void* residual, const float* weight, void* out, float* rstd, int64_t rows, int dim,
                       float eps, int unit, int dtype, hipStream_t st);
int launch_rmsnorm_bwd(const void* x, const float* weight, const float* rstd, const void* dout, void* dx, float* dw, void* ws,
                       int64_t rows, int dim, int unit, int dtype, hipStream_t st);
int launch_ce_rows(void* logits, int64_t pitch, const int64_t* targets, int64_t rows, int vocab, int64_t ignore_index,
                   float softcap, const float* grad_scale, float* lse, float* nll, int write_grad, int dtype, hipStream_t stream);
int launch_transpose(const void* src, void* dst, int64_t rows, int64_t cols, int src_dtype, int dst_dtype, hipStream_t stream);
int launch_ce_valid_count(const int64_t* targets, int64_t n, int64_t ignore_index, int vocab, float* stats, hipStream_t stream);
int launch_ce_loss_reduce(const float* nll, int64_t n, const float* scale, float* loss, hipStream_t stream);

struct AttnArgs {
    ma_tensor4 q, k, v, o, dout, dq, dk, dv;
    float* lse;
    float* delta;
    ma_tile_map map;
    const int64_t* doc;
    int causal;
    int64_t window;
    float scale;
    int B, S, Hq, Hkv, D, T;
    int stages;  // MA_BWD_* mask (backward only)
    // dS^T handed from the dK/dV kernel to the dQ kernel (backward only, may be NULL): bf16
    // [Hq, ds_tiles, 128 kv, 128 q], one 32 KB slot per query head and visited (q tile, kv tile)
    // pair, numbered by map.tile_slot
    void* ds;
    int64_t ds_tiles;
};

// The argument block as the per-item functions of the queue-driven kernels see it: in the constant
// address space (scalar loads), behind a pointer the compiler cannot see through -- and the thread
// id likewise.  Everything derived from either is then computed inside the item that uses it;
// otherwise the compiler hoists all of it out of the loop over items and keeps it in registers
// across the whole loop, which these kernels (512 registers per lane in use) cannot afford.
typedef const __attribute__((address_space(4))) AttnArgs KernArgs;
__device__ __forceinline__ KernArgs& fresh_args() {
    KernArgs* p = (KernArgs*)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(p));
    return *p;
}
__device__ __forceinline__ int fresh_tid() {
    int t = threadIdx.x;
    asm volatile("" : "+v"(t));
    return t;
}

int launch_probe_mfma(int iters, int random_data, int workgroups, unsigned long long* out, hipStream_t st);
int launch_attn_fwd_f32(const AttnArgs& a, hipStream_t st);
int launch_attn_bwd_f32(const AttnArgs& a, hipStream_t st);
int launch_attn_fwd_bf16(const AttnArgs& a, hipStream_t st);
int launch_attn_fwd_pair_bf16(const AttnArgs& a, hipStream_t st);  // even number of q heads per kv head
int launch_attn_bwd_bf16(const AttnArgs& a, hipStream_t st);

// Loads through the scalar cache, waited for on the spot.  For the handful of uniform values a
// workgroup needs before it can request its first tiles: a scalar load has a fraction of a vector
// load's latency and its wait (lgkmcnt) does not queue behind the bulk vector loads already in
// flight.  Load and wait are one asm statement, so the compiler cannot touch the destination
// registers in between.
__device__ __forceinline__ int scalar_load(const int32_t* p) {
    int v;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(p) : "memory");
    return v;
}
__device__ __forceinline__ void scalar_load2(const int32_t* p, const int32_t* q, int& a, int& b) {
    asm volatile("s_load_dword %0, %2, 0x0\n\ts_load_dword %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(a), "=&s"(b) : "s"(p), "s"(q) : "memory");
}

// Workgroup id -> work item.  A unit is a tile row (q tile for the forward and dQ kernels, kv tile
// for the dK/dV kernel) of one batch row; a combo is (unit, kv head) and owns `heads` workgroups
// (the query heads that stream the same K/V, or 1).  Workgroups are handed to the 8 XCDs round-robin
// by id and each XCD has its own L2, so the workgroups of one combo are given ids with the same
// id % 8.  Units are taken in the order of `order` (descending work, from the tile map) so that the
// longest-running workgroups start first; without it, in natural order.  Returns false for the
// padding ids of the last group.
constexpr int kXcds = 8;
__host__ __device__ inline int work_grid(int n_units, int Hkv, int heads) {
    return (n_units * Hkv + kXcds - 1) / kXcds * kXcds * heads;
}
__device__ __forceinline__ bool map_work(int id, int n_units, int T, int Hkv, int heads, const int32_t* order, int& tile,
                                         int& head, int& b) {
    const int x = id % kXcds, n = id / kXcds;
    const int g = n % heads;
    const int c = (n / heads) * kXcds + x;
    if (c >= n_units * Hkv) return false;
    const int rank = c / Hkv, hk = c % Hkv;
    const int u = order ? scalar_load(order + __builtin_amdgcn_readfirstlane(rank)) : rank;
    // (integer division runs on the vector ALU: hand the results back as scalars, so that everything
    // derived from them -- tile-map rows, base pointers -- is addressed and loaded on the scalar side)
    b = __builtin_amdgcn_readfirstlane(u / T);
    tile = __builtin_amdgcn_readfirstlane(u % T);
    head = __builtin_amdgcn_readfirstlane(hk * heads + g);
    return true;
}

// Where the ids handed to map_work come from.  Without counters (ma_tile_map.work_counters NULL) a
// launch has one workgroup per id and each handles its blockIdx.  With counters a launch has one
// workgroup per compute unit and the workgroups pull ids until none is left: id = 8 * k + x, with k
// drawn from counter x -- first the counter of the workgroup's own XCD (blockIdx % 8, which keeps the
// XCD affinity map_work builds into the ids), then, once that one is exhausted, the others'.  Pulling
// keeps the longest-first order of the schedule but lets a compute unit start its next item the
// moment it is done, instead of waiting for the hardware dispatcher's fixed round over the shader
// engines.  The last workgroup to leave puts the counters back to zero for the next launch.
//   counters: kWorkSlot ints per kernel kind (8 queues, then the count of workgroups that have left)
#ifndef MA_LDS
#define MA_LDS __attribute__((address_space(3)))
#endif
constexpr int kWorkSlot = 16;
enum { kQueueFwd = 0, kQueueDq = 1, kQueueDkv = 2 };
struct WorkQueue {
    int32_t* ctr;   // nullptr: one id per workgroup
    int per_xcd;    // ids per queue
    bool first;
    __device__ __forceinline__ void init(int32_t* counters, int kind, int total_ids) {
        ctr = counters ? counters + kind * kWorkSlot : nullptr;
        per_xcd = total_ids / kXcds;
        first = true;
    }
    // The next id, or -1.  Every thread of the workgroup must call it; `box` is one int of LDS that
    // nothing else uses, and a barrier must separate the return from the next call (the kernels
    // end every item with one).
    __device__ __forceinline__ int next(MA_LDS int* box) {
        if (!ctr) {
            const int id = first ? (int)blockIdx.x : -1;
            first = false;
            return id;
        }
        if (threadIdx.x == 0) {
            const int x0 = blockIdx.x % kXcds;
            int id = -1;
            for (int t = 0; t < kXcds && id < 0; ++t) {
                const int x = (x0 + t) % kXcds;
                const int k = atomicAdd(ctr + x, 1);
                if (k < per_xcd) id = k * kXcds + x;
            }
            *box = id;
        }
        __syncthreads();
        return __builtin_amdgcn_readfirstlane(*box);
    }
    __device__ __forceinline__ void leave() {
        if (ctr && threadIdx.x == 0) {
            __threadfence();
            if (atomicAdd(ctr + kXcds, 1) == (int)gridDim.x - 1)
                for (int x = 0; x <= kXcds; ++x) atomicExch(ctr + x, 0);
        }
    }
};
// grid of a launch: one workgroup per id, or (with work queues) at most one per compute unit
inline int compute_units() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    int c = cached[dev];
    if (c <= 0) {
        if (hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || c <= 0) c = 256;
        cached[dev] = c;
    }
    return c;
}
// as many workgroups as the device holds at once (`resident` per compute unit, from the occupancy query)
inline int queue_grid(int total_ids, const int32_t* counters, int resident = 1) {
    if (!counters) return total_ids;
    const int slots = compute_units() * (resident < 1 ? 1 : resident);
    return total_ids < slots ? total_ids : slots;
}
template <typename K>
inline int resident_workgroups(K kernel, int threads, size_t lds_bytes) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, (const void*)kernel, threads, lds_bytes) != hipSuccess || n < 1) n = 1;
    return n;
}

// Walks `reps` times over the concatenation of two tile lists (partial tiles, then full tiles) of a
// tile-map row.  The index of the following entry is always in flight: it is loaded when the current
// one is handed out and only read (readfirstlane) a whole step later, so the walk never waits on
// memory.  Walking backward (full tiles from the highest index down, then the partial ones) makes all
// the workgroups of one document start on the same tile and stay in step, so that they share the
// stream in L2.  `zero` must be a per-lane zero the compiler cannot see through (it keeps the load a plain
// per-lane load whose result stays in a vector register until it is needed).
struct ListWalk {
    const int32_t *pl, *fl;
    int np, n, reps, rep, it;
    int nxt;
    bool backward;  // walk the concatenation from its last entry to its first

    __device__ __forceinline__ int fetch(int c, int zero) const {
        const int i = backward ? n - 1 - c : c;
        return i < np ? pl[i + zero] : fl[i - np + zero];
    }
    __device__ __forceinline__ void init(const int32_t* partial_list, int n_partial, const int32_t* full_list, int n_full,
                                         int repeats, bool reverse) {
        pl = partial_list; fl = full_list; np = n_partial; n = n_partial + n_full; reps = repeats;
        rep = 0; it = -1; backward = reverse;
        nxt = 0;
    }
    // The start of a walk: the entry is loaded and waited for on the spot (uniform address: a scalar
    // load, whose wait does not queue behind the bulk vector loads a kernel has in flight when it
    // starts) -- advance_now() until the first step is found, then prefetch() once; advance() from then on.
    __device__ __forceinline__ bool advance_now(int& tile, bool& partial) {
        if (n == 0) return false;
        if (++it == n) {
            it = 0;
            if (++rep == reps) return false;
        }
        const int i = backward ? n - 1 - it : it;
        tile = scalar_load(i < np ? pl + i : fl + (i - np));
        partial = (backward ? n - 1 - it : it) < np;
        return true;
    }
    __device__ __forceinline__ void prefetch(int zero) {
        if (n) nxt = fetch(it + 1 == n ? 0 : it + 1, zero);
    }
    __device__ __forceinline__ bool advance(int& tile, bool& partial, int zero) {
        if (n == 0) return false;
        if (++it == n) {
            it = 0;
            if (++rep == reps) return false;
        }
        tile = __builtin_amdgcn_readfirstlane(nxt);
        partial = (backward ? n - 1 - it : it) < np;
        nxt = fetch(it + 1 == n ? 0 : it + 1, zero);
        return true;
    }
};
// Steps of STEP rows over a ListWalk of 128-row tiles.  A step is handed out when one of its rows
// can be visible to the workgroup: it starts inside the sequence and, for a partial tile, inside
// [vis_lo, vis_hi] -- the causal / window bounds of the workgroup's own rows folded into two 32-bit
// limits by the caller (full tiles are visible throughout by construction).
constexpr int kNoLimitLo = -0x40000000, kNoLimitHi = 0x7fffffff;
template <int STEP>
struct StepWalk {
    ListWalk walk;
    int zero, half, tile, S, vis_lo, vis_hi;
    int r0;  // first row of the step
    bool partial;

    __device__ __forceinline__ void init(const int32_t* partial_list, int n_partial, const int32_t* full_list, int n_full,
                                         int repeats, bool reverse, int seq_len, int lo, int hi) {
        zero = opaque_lane_zero_();
        walk.init(partial_list, n_partial, full_list, n_full, repeats, reverse);
        half = kTile / STEP - 1; tile = 0; partial = false; S = seq_len; vis_lo = lo; vis_hi = hi; r0 = 0;
    }
    __device__ __forceinline__ static int opaque_lane_zero_() {
        int z;
        asm volatile("v_mov_b32 %0, 0" : "=v"(z));
        return z;
    }
    // the first step of the walk (see ListWalk::advance_now), then next() for the others
    __device__ __forceinline__ bool first() {
        for (;;) {
            if (++half == kTile / STEP) {
                half = 0;
                if (!walk.advance_now(tile, partial)) return false;
            }
            r0 = tile * kTile + half * STEP;
            if ((r0 < S) & (!partial | ((r0 >= vis_lo) & (r0 <= vis_hi)))) {
                walk.prefetch(zero);
                return true;
            }
        }
    }
    __device__ __forceinline__ bool next() {
        for (;;) {
            if (++half == kTile / STEP) {
                half = 0;
                if (!walk.advance(tile, partial, zero)) return false;
            }
            r0 = tile * kTile + half * STEP;
            if ((r0 < S) & (!partial | ((r0 >= vis_lo) & (r0 <= vis_hi)))) return true;
        }
    }
};
// The same walk, resolved ahead of time.  Per step the walk above costs a wave some hundred scalar
// and branch instructions (list bookkeeping, visibility tests, the id-range test of both 32-row
// blocks with its scalar loads), and a wave that has its SIMD to itself pays the full latency of
// every one of them between two MFMA chains.  Here a wave works the steps out 64 at a time, one
// candidate step per lane, and keeps them as one word per step in its own slice of LDS:
//     bits 0..23 first row of the step, 24..28 pass over the lists (the query head of the dK/dV
//     kernel), 29 / 30 the wave has something to do in the second / first 32-row block, 31 partial tile
// so that handing out a step is one LDS word (read a step ahead), a few bit operations and a
// compare.  Every wave of a workgroup derives the same sequence of steps (same inputs); only the
// two block bits are its own.  Filling takes a few vector loads and is needed once per 64 candidates.
// SLOTS: a second word per step, looked up in a table of tile numbers (the compact numbering of the
// visited tiles, ma_tile_map.tile_slot) at slot_base + tile * slot_stride: the backward kernels
// address the dS workspace with it.
template <int STEP, bool SLOTS = false>
struct StepTable {
    static_assert(kTile % STEP == 0 && STEP == 64, "two 32-row blocks per step");
    static constexpr int kPerTile = kTile / STEP;
    const int32_t *pl, *fl;        // partial / full tile lists of the row
    int np, n, reps;
    bool backward;
    int S, vis_lo, vis_hi;         // visibility of a step of a partial tile (the workgroup's rows)
    int blk_lo, blk_hi;            // ... of one of its 32-row blocks (the wave's rows)
    const int64_t* rng;            // (min, max) document id per 32-row block of the batch row, or nullptr
    int64_t own_lo, own_hi;        // id range of the wave's own rows
    MA_LDS uint32_t* slot;         // 64 words of LDS of this wave (with SLOTS: 128, the second half for the tile numbers)
    int total, cbase, cnt, pos;
    uint32_t ahead;                // the entry after the current one (per lane copy of an LDS word)
    const int32_t* slot_tab = nullptr;
    int64_t slot_base = 0, slot_stride = 0;
    uint32_t ahead_slot = 0;
    int tile_slot = -1;            // of the current step (SLOTS)
    uint32_t slot_last = 0;        // the last slot of the workspace: numbers are clamped to it (a stale count must not read past the end)
    __device__ __forceinline__ void numbering(const int32_t* table, int64_t base, int64_t stride, int64_t slots) {
        slot_tab = table; slot_base = base; slot_stride = stride; slot_last = (uint32_t)(slots - 1);
    }

    __device__ __forceinline__ void init(const int32_t* partial_list, int n_partial, const int32_t* full_list, int n_full,
                                         int repeats, bool reverse, int seq_len, int lo, int hi, int wave_lo, int wave_hi,
                                         const int64_t* block_ranges, int64_t own_min, int64_t own_max, MA_LDS uint32_t* lds_slot) {
        pl = partial_list; fl = full_list; np = n_partial; n = n_partial + n_full; reps = repeats; backward = reverse;
        S = seq_len; vis_lo = lo; vis_hi = hi; blk_lo = wave_lo; blk_hi = wave_hi;
        rng = block_ranges; own_lo = own_min; own_hi = own_max; slot = lds_slot;
        total = n * kPerTile * repeats; cbase = 0; cnt = 0; pos = 0; ahead = 0;
        r0 = 0; rep = 0; partial = act0 = act1 = false;
    }
    // works out candidates cbase .. cbase + 63 and keeps the visible ones; returns how many
    __device__ __forceinline__ int fill() {
        const int lane = __lane_id();
        const int c = cbase + lane;
        const bool valid = c < total;
        const int per_pass = n * kPerTile;
        const int cc = valid ? c : 0;
        const int rep = cc / per_pass, wi = cc - rep * per_pass;
        const int it = wi / kPerTile, half = wi - it * kPerTile;
        const int idx = backward ? n - 1 - it : it;
        const bool partial = idx < np;
        int tile = 0;
        if (valid) tile = partial ? pl[idx] : fl[idx - np];
        const int r0 = tile * kTile + half * STEP;
        const bool vis = valid & (r0 < S) & (!partial | ((r0 >= vis_lo) & (r0 <= vis_hi)));
        bool act0 = block_inside(r0, partial), act1 = block_inside(r0 + 32, partial);
        if (rng && partial && vis) {  // no row of the block shares a document with the wave's own rows
            const int64_t* e = rng + (size_t)(r0 / 32) * 2;
            act0 &= (e[0] <= own_hi) & (e[1] >= own_lo);
            act1 &= (e[2] <= own_hi) & (e[3] >= own_lo);
        }
        const uint32_t word = (uint32_t)r0 | ((uint32_t)rep << 24) | ((uint32_t)act1 << 29) | ((uint32_t)act0 << 30) | ((uint32_t)partial << 31);
        const uint64_t mask = __ballot(vis);
        const int at = __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
        if (vis) slot[at] = word;
        if constexpr (SLOTS) {
            if (vis && slot_tab) slot[64 + at] = min((uint32_t)slot_tab[slot_base + (int64_t)tile * slot_stride], slot_last);
        }
        cbase += 64;
        return __builtin_popcountll(mask);
    }
    __device__ __forceinline__ bool block_inside(int r0, bool partial) const {
        return (r0 < S) & (!partial | ((r0 >= blk_lo) & (r0 <= blk_hi)));
    }
    // the next 64 candidates that hold a step at all; false when the walk is over.  prime() right
    // after init(): the loads of the first fill are then ahead of whatever the kernel requests next.
    __device__ __forceinline__ bool refill() {
        cnt = 0;
        while (cnt == 0 && cbase < total) cnt = fill();
        pos = 0;
        ahead = slot[0];
        if constexpr (SLOTS) ahead_slot = slot[64];
        return cnt != 0;
    }
    __device__ __forceinline__ void prime() { refill(); }
    // Moves on to the next step (false when the walk is over): its first row, the pass over the
    // lists it belongs to, the kind of its tile, and whether this wave has work in its two blocks.
    int r0, rep;
    bool partial, act0, act1;
    __device__ __forceinline__ bool next() {
        if (pos == cnt && !refill()) return false;
        const uint32_t word = __builtin_amdgcn_readfirstlane(ahead);
        if constexpr (SLOTS) tile_slot = (int)__builtin_amdgcn_readfirstlane(ahead_slot);
        ++pos;
        ahead = slot[pos & 63];  // read now, used at the next call
        if constexpr (SLOTS) ahead_slot = slot[64 + (pos & 63)];
        r0 = (int)(word & 0xffffffu);
        rep = (int)((word >> 24) & 31u);
        act1 = (word >> 29) & 1u;
        act0 = (word >> 30) & 1u;
        partial = (word >> 31) != 0;
        return true;
    }
};

// the same test for a block of rows starting at r0 (bounds of the wave's own rows)
__device__ __forceinline__ bool block_visible(int r0, int S, bool partial, int lo, int hi) {
    return (r0 < S) & (!partial | ((r0 >= lo) & (r0 <= hi)));
}
// Visibility limits for a walk over kv rows by query rows [q_lo, q_hi] (kv_side = false) or over
// query rows by kv rows [k_lo, k_hi] (kv_side = true), for steps/blocks of `rows` rows.
__device__ __forceinline__ void visibility_limits(bool kv_side, int own_lo, int own_hi, int rows, bool bounded, int wlim,
                                                  bool windowed, int& lo, int& hi) {
    if (!kv_side) {  // kv block [r0, r0+rows): needs r0 <= q_hi (kv <= q) and r0 + rows - 1 >= q_lo - window
        hi = bounded ? own_hi : kNoLimitHi;
        lo = windowed ? own_lo - wlim - (rows - 1) : kNoLimitLo;
    } else {         // q block [r0, r0+rows): needs r0 + rows - 1 >= k_lo (q >= kv) and r0 <= k_hi + window
        lo = bounded ? own_lo - (rows - 1) : kNoLimitLo;
        hi = windowed ? own_hi + wlim : kNoLimitHi;
    }
}

// ---- document-id ranges of 32-row blocks (ma_tile_map.block_doc_range) ---------------------------
// Fetched with scalar loads (plain reads through the scalar cache): the data is workgroup-uniform.
// A load is issued early (load_*) and waited for just before its first use (ready()).
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x8_t __attribute__((ext_vector_type(8)));
struct DocRange {      // one block
    i32x4_t raw;
    __device__ __forceinline__ void load(const int64_t* entry) { asm volatile("s_load_dwordx4 %0, %1, 0x0" : "=s"(raw) : "s"(entry)); }
    __device__ __forceinline__ void ready() { asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(raw)); }
    __device__ __forceinline__ int64_t lo() const { return (int64_t)(((uint64_t)(uint32_t)raw[1] << 32) | (uint32_t)raw[0]); }
    __device__ __forceinline__ int64_t hi() const { return (int64_t)(((uint64_t)(uint32_t)raw[3] << 32) | (uint32_t)raw[2]); }
};
// two list lengths and one block's id range in one round trip: the three loads and their wait are one
// asm statement (a load left in flight across other code could land in registers the compiler has
// meanwhile given to something else)
__device__ __forceinline__ void scalar_load2_range(const int32_t* p, const int32_t* q, const int64_t* entry, int& a, int& b, DocRange& r) {
    asm volatile("s_load_dword %0, %3, 0x0\n\ts_load_dword %1, %4, 0x0\n\ts_load_dwordx4 %2, %5, 0x0\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(a), "=&s"(b), "=&s"(r.raw) : "s"(p), "s"(q), "s"(entry) : "memory");
}
struct DocRange2 {     // two consecutive blocks (one 64-row step)
    i32x8_t raw;
    __device__ __forceinline__ void load(const int64_t* entry) { asm volatile("s_load_dwordx8 %0, %1, 0x0" : "=s"(raw) : "s"(entry)); }
    __device__ __forceinline__ void ready() { asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(raw)); }
    __device__ __forceinline__ int64_t lo(int k) const { return (int64_t)(((uint64_t)(uint32_t)raw[4 * k + 1] << 32) | (uint32_t)raw[4 * k]); }
    __device__ __forceinline__ int64_t hi(int k) const { return (int64_t)(((uint64_t)(uint32_t)raw[4 * k + 3] << 32) | (uint32_t)raw[4 * k + 2]); }
    // can block k share a document with rows whose ids span [own_lo, own_hi]?
    __device__ __forceinline__ bool meets(int k, int64_t own_lo, int64_t own_hi) const { return (int)(lo(k) <= own_hi) & (int)(hi(k) >= own_lo); }
};

__device__ __forceinline__ int opaque_lane_zero() {
    int z;
    asm volatile("v_mov_b32 %0, 0" : "=v"(z));
    return z;
}

inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(MA_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return MA_OK;
}

}  // namespace ma
