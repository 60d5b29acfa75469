// Block-sparse tile map from document_ids, in torch's BlockMask format.
//
// Stands in for create_block_mask(make_document_mask_wrapper(...), B, None, S, S)
// (maester/models/gemma/model.py:694-730), which materialises a [B,1,S,S] bool and block-reduces
// it (torch/nn/attention/flex_attention.py:979-1022, 429-441).  Here every 128x128 tile is
// classified from the document ids of the two 128-row slices it covers (exact for arbitrary ids,
// no S^2 memory): first by their (min, max) id ranges, and only the tiles the ranges cannot settle
// by an exact 128x128 count; then the ordered lists are emitted: set tiles ascending, unset tiles
// ascending.
#include "common.h"

#include <mutex>

namespace ma {

// class codes in the workspace: 0 empty, 1 partial, 2 full

// (min, max) document id over the valid rows of every 128-row tile; one wave per tile.  Also clears
// the counter of the hard-tile list.  With doc == nullptr only the counter is cleared.
__global__ __launch_bounds__(256) void tile_ranges_kernel(const int64_t* __restrict__ doc, int B, int S, int T,
                                                          int64_t* __restrict__ rng, int* __restrict__ n_hard,
                                                          int32_t* __restrict__ work_counters) {
    if (blockIdx.x == 0 && threadIdx.x == 0) *n_hard = 0;
    if (blockIdx.x == 0 && work_counters && threadIdx.x < MA_WORK_COUNTERS) work_counters[threadIdx.x] = 0;
    const int tile = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (!doc || tile >= B * T) return;
    const int b = tile / T, r0 = (tile % T) * kTile;
    const int64_t* row = doc + (size_t)b * S;
    const int last = S - 1;
    int64_t lo = row[min(r0 + lane, last)], hi = lo;
    const int64_t x = row[min(r0 + 64 + lane, last)];
    lo = min(lo, x);
    hi = max(hi, x);
    for (int off = 32; off > 0; off >>= 1) {
        lo = min(lo, __shfl_xor(lo, off, 64));
        hi = max(hi, __shfl_xor(hi, off, 64));
    }
    if (lane == 0) {
        rng[(size_t)tile * 2] = lo;
        rng[(size_t)tile * 2 + 1] = hi;
    }
}

// One thread per tile.  Most tiles are settled without looking at a single pair:
//   * ruled out by the causal / window bound, or by disjoint document-id ranges      -> empty
//   * both tiles hold one and the same document, every pair passes the bound, and the tile lies
//     inside the sequence                                                              -> full
// The rest (the diagonal, tiles a document boundary runs through, ragged edges) go on a list and are
// counted exactly by count_hard_tiles_kernel.
__global__ __launch_bounds__(256) void classify_easy_kernel(const int64_t* __restrict__ rng, int has_doc, int B, int S, int T,
                                                             int causal, int64_t window, uint8_t* __restrict__ cls,
                                                             int* __restrict__ n_hard, int32_t* __restrict__ hard) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)B * T * T) return;
    const int j = (int)(idx % T), i = (int)((idx / T) % T), b = (int)(idx / ((int64_t)T * T));
    const int q0 = i * kTile, k0 = j * kTile;
    const bool bounded = causal || window >= 0;
    bool dead = bounded && k0 > q0 + kTile - 1;
    if (window >= 0 && (int64_t)q0 - (int64_t)(k0 + kTile - 1) > window) dead = true;
    int c = -1;  // undecided
    if (dead) c = 0;
    else if (has_doc) {
        const int64_t* rrow = rng + (size_t)b * T * 2;
        const int64_t qlo = rrow[2 * i], qhi = rrow[2 * i + 1], klo = rrow[2 * j], khi = rrow[2 * j + 1];
        if (klo > qhi || khi < qlo) c = 0;
        else if (klo == khi && qlo == qhi && klo == qlo) c = -2;  // one document on both sides
    } else c = -2;                                                // no document term
    if (c == -2) {
        bool all = q0 + kTile <= S && k0 + kTile <= S;
        if (bounded && !(q0 >= k0 + kTile - 1)) all = false;
        if (window >= 0 && (int64_t)(q0 + kTile - 1) - (int64_t)k0 > window) all = false;
        c = all ? 2 : -1;
    }
    if (c >= 0) cls[idx] = (uint8_t)c;
    else hard[atomicAdd(n_hard, 1)] = (int32_t)idx;
}

// Exact class of the listed tiles: 128 x 128 compares from the two 128-id slices, as torch's dense
// mask would give.  One workgroup per listed tile (grid-stride over the list).
__global__ __launch_bounds__(kTile) void count_hard_tiles_kernel(const int64_t* __restrict__ doc, int S, int T, int causal,
                                                                 int64_t window, uint8_t* __restrict__ cls,
                                                                 const int* __restrict__ n_hard,
                                                                 const int32_t* __restrict__ hard) {
    __shared__ int64_t kdoc[kTile];
    __shared__ int wave_cnt[kTile / 64];
    const int t = threadIdx.x;
    const int n = *n_hard;
    for (int e = blockIdx.x; e < n; e += gridDim.x) {
        const int64_t idx = hard[e];
        const int j = (int)(idx % T), i = (int)((idx / T) % T), b = (int)(idx / ((int64_t)T * T));
        const int q0 = i * kTile, k0 = j * kTile;
        const int64_t* drow = doc ? doc + (size_t)b * S : nullptr;
        if (drow) kdoc[t] = (k0 + t < S) ? drow[k0 + t] : 0;
        __syncthreads();
        const int q = q0 + t;
        int cnt = 0;
        if (q < S) {
            const int64_t dq = drow ? drow[q] : 0;
            const int kmax = min(kTile, S - k0);
            for (int c = 0; c < kmax; ++c) {
                bool ok = pair_allowed(q, k0 + c, causal, window);
                if (drow) ok = ok && (kdoc[c] == dq);
                cnt += ok ? 1 : 0;
            }
        }
        for (int off = 32; off > 0; off >>= 1) cnt += __shfl_down(cnt, off, 64);
        if ((t & 63) == 0) wave_cnt[t >> 6] = cnt;
        __syncthreads();
        if (t == 0) {
            int total = 0;
            for (int w = 0; w < kTile / 64; ++w) total += wave_cnt[w];
            cls[idx] = total == 0 ? 0 : (total == kTile * kTile ? 2 : 1);
        }
        __syncthreads();
    }
}

// One wave per (list kind, batch row, tile row).  kind: 0 kv partial, 1 kv full, 2 q partial, 3 q full.
__global__ __launch_bounds__(64) void order_lists_kernel(const uint8_t* __restrict__ cls, int T, ma_tile_map out) {
    const int r = blockIdx.x, b = blockIdx.y, kind = blockIdx.z;
    const int lane = threadIdx.x;
    const uint8_t want = (kind & 1) ? 2 : 1;
    const bool transposed = kind >= 2;
    const uint8_t* base = cls + (size_t)b * T * T;
    int32_t* num = kind == 0 ? out.kv_num_blocks : kind == 1 ? out.full_kv_num_blocks
                 : kind == 2 ? out.q_num_blocks : out.full_q_num_blocks;
    int32_t* idx = kind == 0 ? out.kv_indices : kind == 1 ? out.full_kv_indices
                 : kind == 2 ? out.q_indices : out.full_q_indices;
    num += (size_t)b * T + r;
    idx += ((size_t)b * T + r) * T;

    int total = 0;
    for (int c0 = 0; c0 < T; c0 += 64) {
        const int c = c0 + lane;
        bool set = false;
        if (c < T) set = (transposed ? base[(size_t)c * T + r] : base[(size_t)r * T + c]) == want;
        total += __popcll(__ballot(set));
    }
    int seen_set = 0;
    for (int c0 = 0; c0 < T; c0 += 64) {
        const int c = c0 + lane;
        bool set = false;
        if (c < T) set = (transposed ? base[(size_t)c * T + r] : base[(size_t)r * T + c]) == want;
        const unsigned long long m = __ballot(set);
        const int before = __popcll(m & ((1ull << lane) - 1ull));
        if (c < T) {
            const int set_before = seen_set + before;
            const int pos = set ? set_before : total + (c - set_before);
            idx[pos] = c;
        }
        seen_set += __popcll(m);
    }
    if (lane == 0) *num = total;
}

// Compact numbering of the visited tiles: one wave per tile row (b, i).  The row's first slot is the
// number of visited tiles in the rows before it (summed from the list lengths, B*T terms at most);
// inside the row the visited tiles are numbered by ascending j.  The last row also leaves the total.
__global__ __launch_bounds__(64) void tile_slots_kernel(const uint8_t* __restrict__ cls, int rows, int T, ma_tile_map out) {
    const int row = blockIdx.x, lane = threadIdx.x;
    int before = 0;
    for (int r = lane; r < row; r += 64) before += out.kv_num_blocks[r] + out.full_kv_num_blocks[r];
    for (int off = 32; off > 0; off >>= 1) before += __shfl_xor(before, off, 64);
    const uint8_t* base = cls + (size_t)row * T;
    int32_t* dst = out.tile_slot + (size_t)row * T;
    int seen = 0;
    for (int c0 = 0; c0 < T; c0 += 64) {
        const int c = c0 + lane;
        const bool set = c < T && base[c] != 0;
        const unsigned long long m = __ballot(set);
        if (c < T) dst[c] = set ? before + seen + __popcll(m & ((1ull << lane) - 1ull)) : -1;
        seen += __popcll(m);
    }
    if (row == rows - 1 && lane == 0 && out.tile_count) *out.tile_count = before + seen;
}

// Launch schedule: the B*T tile rows ordered by descending work (number of tiles in the row's lists,
// partial + full), ties by ascending index.  Block 0 orders the q tiles by their kv lists, block 1
// the kv tiles by their q lists.  Rank by counting: N is small (B*T), the keys sit in LDS.
constexpr int kSchedMax = 8192;
__global__ __launch_bounds__(1024) void schedule_kernel(int N, ma_tile_map out) {
    __shared__ int key[kSchedMax];
    const bool qside = blockIdx.x == 0;
    int32_t* dst = qside ? out.q_tile_order : out.kv_tile_order;
    if (!dst) return;
    if (N > kSchedMax) {  // too many rows to rank here: natural order
        for (int e = threadIdx.x; e < N; e += blockDim.x) dst[e] = e;
        return;
    }
    const int32_t* na = qside ? out.kv_num_blocks : out.q_num_blocks;
    const int32_t* nb = qside ? out.full_kv_num_blocks : out.full_q_num_blocks;
    for (int e = threadIdx.x; e < N; e += blockDim.x) key[e] = na[e] + nb[e];
    __syncthreads();
    for (int e = threadIdx.x; e < N; e += blockDim.x) {
        const int k = key[e];
        int rank = 0;
        for (int f = 0; f < N; ++f) rank += (key[f] > k) | ((key[f] == k) & (f < e));
        dst[rank] = e;
    }
}

// (min, max) document id of every block of MA_DOC_BLOCK rows; one half-wave per block.
__global__ __launch_bounds__(256) void block_ranges_kernel(const int64_t* __restrict__ doc, int B, int S, int NB,
                                                           int64_t* __restrict__ out) {
    const int blk = blockIdx.x * 8 + threadIdx.x / MA_DOC_BLOCK;  // 8 blocks per workgroup
    const int l = threadIdx.x % MA_DOC_BLOCK;
    if (blk >= B * NB) return;
    const int b = blk / NB, r0 = (blk % NB) * MA_DOC_BLOCK;
    const int row = min(r0 + l, S - 1);  // rows past the end repeat the last one
    int64_t lo = doc[(size_t)b * S + row], hi = lo;
    for (int off = MA_DOC_BLOCK / 2; off > 0; off >>= 1) {
        const int64_t olo = __shfl_xor(lo, off, MA_DOC_BLOCK), ohi = __shfl_xor(hi, off, MA_DOC_BLOCK);
        lo = min(lo, olo);
        hi = max(hi, ohi);
    }
    if (l == 0) {
        out[(size_t)blk * 2] = lo;
        out[(size_t)blk * 2 + 1] = hi;
    }
}

int launch_tile_map(const int64_t* doc, int B, int S, int causal, int64_t window, const ma_tile_map& out,
                    void* ws, hipStream_t st) {
    const int T = (S + kTile - 1) / kTile;
    // workspace: class bytes | tile id ranges | hard-tile counter | hard-tile list
    uint8_t* cls = (uint8_t*)ws;
    const size_t ntiles = (size_t)B * T * T;
    int64_t* rng = (int64_t*)((char*)ws + ((ntiles + 15) & ~(size_t)15));
    int* n_hard = (int*)(rng + (size_t)B * T * 2);
    int32_t* hard = (int32_t*)((char*)n_hard + 16);
    hipLaunchKernelGGL(tile_ranges_kernel, dim3((B * T + 3) / 4), dim3(256), 0, st, doc, B, S, T, rng, n_hard,
                       out.work_counters);
    int rc = check_launch("tile_ranges_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(classify_easy_kernel, dim3((unsigned)((ntiles + 255) / 256)), dim3(256), 0, st, rng, doc ? 1 : 0, B, S, T,
                       causal, window, cls, n_hard, hard);
    rc = check_launch("classify_easy_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(count_hard_tiles_kernel, dim3((unsigned)(ntiles < 4096 ? ntiles : 4096)), dim3(kTile), 0, st, doc, S, T,
                       causal, window, cls, n_hard, hard);
    rc = check_launch("count_hard_tiles_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(order_lists_kernel, dim3(T, B, 4), dim3(64), 0, st, cls, T, out);
    rc = check_launch("order_lists_kernel");
    if (rc) return rc;
    if (out.tile_slot) {
        hipLaunchKernelGGL(tile_slots_kernel, dim3(B * T), dim3(64), 0, st, cls, B * T, T, out);
        rc = check_launch("tile_slots_kernel");
        if (rc) return rc;
    }
    if (doc && out.block_doc_range) {
        const int NB = 2 * ((S + 63) / 64);
        hipLaunchKernelGGL(block_ranges_kernel, dim3((B * NB + 7) / 8), dim3(256), 0, st, doc, B, S, NB, out.block_doc_range);
        rc = check_launch("block_ranges_kernel");
        if (rc) return rc;
    }
    if (!out.q_tile_order && !out.kv_tile_order) return rc;
    hipLaunchKernelGGL(schedule_kernel, dim3(2), dim3(1024), 0, st, B * T, out);
    return check_launch("schedule_kernel");
}

// ---- the build without a caller-provided workspace ----------------------------------------------------
// Device scratch owned by the library: every GPU the library runs on holds its own copy of this array
// until the process ends.  In host code the array's name is only a handle; its address on the current
// device comes from hipGetSymbolAddress, once per device, and that pointer is what the kernels get.
static __device__ __align__(256) unsigned char scratch[MA_TILE_MAP_STATIC_BYTES];

static void* g_scratch_ptr[64];          // per device, written once under g_scratch_lock
static std::mutex g_scratch_lock;

int static_tile_map_scratch(void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(MA_ERR_LAUNCH, "ma_tile_map_build_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= 64) return fail(MA_ERR_UNSUPPORTED, "ma_tile_map_build_static: device index %d (at most 64 devices)", dev);
    std::lock_guard<std::mutex> guard(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(MA_ERR_LAUNCH, "ma_tile_map_build_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return MA_OK;
}

}  // namespace ma
