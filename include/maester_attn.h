/* maester_attn.h -- C ABI of the MI355X (gfx950) packed-SFT document-masked attention path.
 *
 * The library replaces, for maester's Gemma attention, everything between the qkv split and
 * o_proj (maester/models/gemma/model.py:364-439) plus the per-step BlockMask construction
 * (model.py:694-730).  The reference is pure Python on torch, so there is no FFI to mirror; each
 * entry point below cites the reference code it stands in for.
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer owned by the caller (torch); the library allocates nothing,
 *    never synchronises and never throws.  Work is enqueued on `stream` (a hipStream_t passed as
 *    void*; NULL = the default stream).
 *  - Host-side state of the library: the thread-local message behind ma_last_error(), a per-device
 *    cache of the compute-unit count and of each kernel's occupancy (read-only after first use) and,
 *    for ma_tile_map_build_static alone, the per-device address of its scratch array.  Device-side
 *    state: that scratch array, and the work counters inside a caller's ma_tile_map (see there).
 *  - Every function returns MA_OK (0) or a negative MA_ERR_* code; the message of the last error of
 *    the calling thread is available from ma_last_error().  Arguments are validated before any
 *    launch, so the error paths run on a host without a GPU.
 *  - Activations are addressed as x[b, s, h, d] = base + b*stride_b + s*stride_s + h*stride_h + d
 *    (strides in ELEMENTS, last dim contiguous), which covers both the [B,S,H,D] views of the fused
 *    qkv projection output (model.py:358-364) and [B,H,S,D] tensors.
 *  - Tile lists use torch's BlockMask format with 128x128 tiles and a head dim of 1:
 *    *_num_blocks int32 [B, T], *_indices int32 [B, T, T], T = ceil(S/128).
 */
#ifndef MAESTER_ATTN_H
#define MAESTER_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MA_OK 0
#define MA_ERR_BAD_ARG (-1)
#define MA_ERR_UNSUPPORTED (-2)
#define MA_ERR_LAUNCH (-3)

#define MA_DTYPE_F32 0
#define MA_DTYPE_BF16 1

#define MA_TILE 128 /* BlockMask tile edge (torch _DEFAULT_SPARSE_BLOCK_SIZE) */
#define MA_DOC_BLOCK 32 /* rows per entry of ma_tile_map.block_doc_range */
#define MA_WORK_COUNTERS 64 /* ints in ma_tile_map.work_counters */

/* Version of this header (major*10000 + minor*100 + patch).  It changes whenever a struct or a
 * signature below changes; ma_version() returns the value the library was built with, and a caller
 * built against another header must not go on (its ma_tile_map has another layout). */
#define MA_ABI_VERSION 10200
int ma_version(void);

/* Message describing the last error returned to the calling thread ("" if none). */
const char* ma_last_error(void);

/* Strided [B,S,H,D] activation descriptor (strides in elements). */
typedef struct ma_tensor4 {
    void* ptr;
    int64_t stride_b, stride_s, stride_h;
} ma_tensor4;

/* The eight BlockMask tensors (torch/nn/attention/flex_attention.py BlockMask). */
typedef struct ma_tile_map {
    int32_t* kv_num_blocks;      /* [B,T]   partial tiles per q-tile row            */
    int32_t* kv_indices;         /* [B,T,T] partial kv tiles ascending, then the rest */
    int32_t* full_kv_num_blocks; /* [B,T]   full tiles per q-tile row               */
    int32_t* full_kv_indices;    /* [B,T,T]                                          */
    int32_t* q_num_blocks;       /* [B,T]   the same four on the transposed tile matrix */
    int32_t* q_indices;          /* [B,T,T]                                          */
    int32_t* full_q_num_blocks;  /* [B,T]                                            */
    int32_t* full_q_indices;     /* [B,T,T]                                          */
    /* Launch schedules (not part of BlockMask): the B*T q tiles (b*T + i) ordered by descending
     * number of visited kv tiles, and the B*T kv tiles ordered by descending number of visiting q
     * tiles.  The attention kernels start the longest-running tiles first.  Either may be NULL
     * (natural order). */
    int32_t* q_tile_order;       /* [B*T] */
    int32_t* kv_tile_order;      /* [B*T] */
    /* Document-id range (min, max) of every block of MA_DOC_BLOCK consecutive rows (not part of
     * BlockMask either): inside a partial tile the kernels skip the 32x32 sub-blocks whose q rows
     * and kv rows have disjoint id ranges -- no pair of them can share a document.  May be NULL, and
     * is ignored when document_ids is NULL (then nothing is skipped on that ground). */
    int64_t* block_doc_range;    /* [B, 2 * ceil(S / 64), 2]: blocks past the end repeat the last row */
    /* Work queues of the attention kernels (not part of BlockMask): MA_WORK_COUNTERS ints that
     * ma_tile_map_build zeroes.  With it, a kernel is launched as one workgroup per compute unit and
     * the workgroups pull work items (in the order of the launch schedules) until none is left, which
     * keeps every compute unit busy to the end; the last workgroup of a launch puts the counters back
     * to zero.  Launches that share a tile map must therefore be ordered (same stream, or events):
     * two of them running at once would share the counters.  May be NULL: then one workgroup is
     * launched per work item, as many as there are, and the hardware dispatcher places them. */
    int32_t* work_counters;      /* [MA_WORK_COUNTERS] */
    /* Compact numbering of the visited tiles (not part of BlockMask): tile_slot[b,i,j] = rank of tile
     * (q tile i, kv tile j) of batch row b among the visited (partial or full) tiles of the whole map in
     * (b, i, j) order, -1 for a tile that is never visited; tile_count[0] = their number.  The backward
     * indexes the dS workspace with it, which then holds visited tiles only.  Both may be NULL (no dS
     * hand-over).  visited_tiles is the HOST copy of tile_count[0] that sizes that workspace: the
     * caller reads it back once per map (one synchronisation per training step, the map being shared
     * by all layers), or leaves 0: then the backward recomputes instead of handing dS over.  It must
     * be the count of THIS build of the map (read after the build has run, on the build's stream): the
     * kernels clamp every slot number to visited_tiles - 1, so a stale or too small value cannot make
     * them touch memory past the workspace, but the gradients of such a call are undefined. */
    int32_t* tile_slot;          /* [B,T,T] */
    int32_t* tile_count;         /* [1] */
    int64_t visited_tiles;       /* host value */
} ma_tile_map;

/* ---- device probe (measurement support; no counterpart in the reference) ---------------------------
 * Runs `workgroups` workgroups of four waves (one per SIMD) that each issue 16 * iters
 * v_mfma_f32_32x32x16_bf16 back to back on two accumulators, with operands of all ones or
 * (random_data) pseudo-random values in [-1, 1].  out (device, three uint64): shader clocks and ticks
 * of the constant 100 MHz counter that the first wave spent in the loop, and a flag that keeps the
 * chain alive.  bench.py --probe turns them into the clock the GPU holds under that load and the
 * MFMA rate that any kernel could sustain at most. */
int ma_probe_mfma(int iters, int random_data, int workgroups, uint64_t* out, void* stream);

/* ---- block-sparse tile map --------------------------------------------------------------------
 * Replaces create_block_mask(make_document_mask_wrapper(base, document_ids), B, None, S, S)
 * (maester/models/gemma/model.py:694-706 global, 714-730 local; torch
 * flex_attention.py:979-1022 tile counts, 429-441 ordered lists).  Predicate:
 *   same_doc(q,kv) && (!causal || q >= kv) && (window < 0 || (q >= kv && q - kv <= window)).
 * document_ids: int64 [B,S] contiguous, or NULL (no document term; model.py:227-228).
 * workspace: at least ma_tile_map_workspace_bytes(B,S) bytes of device scratch.
 * Output is bit-exact with torch's BlockMask tensors, including the list tails. */
size_t ma_tile_map_workspace_bytes(int B, int S);
int ma_tile_map_build(const int64_t* document_ids, int B, int S, int causal, int64_t window,
                      const ma_tile_map* out, void* workspace, size_t workspace_bytes, void* stream);

/* The same build for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): no workspace argument; the scratch is a fixed array of
 * MA_TILE_MAP_STATIC_BYTES that the library holds in device memory on every GPU it runs on until the
 * process ends.  No counterpart in the reference.  The call allocates nothing and frees nothing;
 * (B, S) whose ma_tile_map_workspace_bytes exceeds MA_TILE_MAP_STATIC_BYTES are rejected with
 * MA_ERR_UNSUPPORTED (4 MiB covers B*ceil(S/128)^2 <= ~830 000 tiles, e.g. B=8 at S=32768).
 * Every call on one GPU uses that GPU's one array (nothing in it needs to survive between calls or to
 * be cleared by the caller): calls that overlap on one GPU -- two streams, two threads -- race; order
 * them on one stream or with events.  Same outputs as ma_tile_map_build, bit for bit. */
#define MA_TILE_MAP_STATIC_BYTES (4u << 20)
int ma_tile_map_build_static(const int64_t* document_ids, int B, int S, int causal, int64_t window,
                             const ma_tile_map* out, void* stream);

/* ---- ids of packed rows ----------------------------------------------------------------------------
 * Replaces PackedSFTDataset._generate_position_ids / _generate_document_ids
 * (maester/sft/packed_dataset.py:138-185) and their stacking in packed_collate_fn
 * (maester/sft/dataset.py:198-220), on the device: the i-th boundary (start, length) of row b covers
 * tokens [start, min(start + length, S)) with positions 0, 1, ... and document id i; a later
 * boundary overwrites an earlier one; uncovered tokens (padding) get position 0 and id -1.
 * starts, lengths: int32 [B, max_docs] (row-major, entries past counts[b] ignored); counts: int32 [B].
 * position_ids, document_ids: int64 [B,S] outputs; either may be NULL. */
int ma_packed_ids_build(const int32_t* starts, const int32_t* lengths, const int32_t* counts, int B, int max_docs, int S,
                        int64_t* position_ids, int64_t* document_ids, void* stream);

/* ---- sandwich RMSNorms of the decoder layer ----------------------------------------------------------
 * Replaces RMSNorm.forward (maester/models/gemma/model.py:135-172) as Gemma2DecoderLayer.forward uses
 * it (model.py:488-508), and its autograd:
 *   r = rsqrt(mean(x^2) + eps);  y = x * r * (add_unit_offset ? 1 + w : w)     (fp32 math)
 *   out = residual ? residual + round(y) : y        (round = cast to the IO dtype, as the reference
 *         does between the post-norm and `residual + hidden_states`).
 * x, residual, out, dout, dx: contiguous [rows, dim] of dtype; weight, dweight: fp32 [dim];
 * rstd: fp32 [rows] (forward output, may be NULL when no backward follows; backward input).
 * The gradient of the residual input is dout itself (nothing to compute).  dim: a multiple of 8, at
 * most 8192.  out may alias x or residual; dx may alias dout. */
size_t ma_rmsnorm_bwd_workspace_bytes(int64_t rows, int dim);
int ma_rmsnorm_fwd(const void* x, const void* residual, const float* weight, void* out, float* rstd, int64_t rows, int dim,
                   float eps, int add_unit_offset, int dtype, void* stream);
int ma_rmsnorm_bwd(const void* x, const float* weight, const float* rstd, const void* dout, void* dx, float* dweight,
                   void* workspace, size_t workspace_bytes, int64_t rows, int dim, int add_unit_offset, int dtype, void* stream);

/* ---- softmax cross entropy of the fused linear + cross-entropy loss ------------------------------------
 * Replaces the elementwise half of linear_cross_entropy(hidden.flatten(0,1), embedder_weight,
 * labels.flatten(0,1)) (maester/models/gemma/model.py:762-769; cut-cross-entropy 25.9.3, defaults:
 * ignore_index -100, mean over the rows that count) and of F.cross_entropy(pred.float(), labels)
 * (train.py:258-259).  The caller forms the logits a block of rows at a time (library GEMM), calls
 * ma_ce_rows on the block and uses what it leaves there for the two gradient GEMMs.
 *
 * ma_ce_valid_count: stats[0] = number of targets that count (!= ignore_index, inside [0, vocab)),
 *   stats[1] = 1 / stats[0] (the gradient scale of the mean reduction), both fp32 on the device.
 * ma_ce_rows: logits [rows, vocab] of dtype with `pitch` elements between rows; targets int64 [rows].
 *   Per row: lse[row] = log sum_j exp(x_j); nll[row] = lse - x_label, 0 for a row that does not count
 *   (natural log, fp32; either output may be NULL).  softcap > 0 replaces x by softcap*tanh(x/softcap).
 *   With write_grad the row is overwritten by (softmax(x) - onehot(label)) * grad_scale[0] (times the
 *   soft cap's derivative), zeros for a row that does not count; grad_scale: device fp32 or NULL (= 1).
 * ma_ce_loss_reduce: loss[0] = (sum of nll[0..n) in a fixed order) * scale[0]; scale device fp32 or
 *   NULL (= 1).  With scale = stats + 1 and no row that counts the loss is NaN, as torch's is.
 * ma_transpose: dst[c, r] = src[r, c] for contiguous src [rows, cols] of src_dtype and dst [cols, rows]
 *   of dst_dtype: the same dtype (the copy of the classifier that is contiguous along the
 *   vocabulary, for the d hidden GEMM) or fp32 -> bf16 (the weight gradient, summed over row blocks
 *   in fp32 as [K, V], handed back as [V, K] in the activation dtype); rows <= 65535 * 64. */
int ma_ce_valid_count(const int64_t* targets, int64_t n, int64_t ignore_index, int64_t vocab, float* stats, void* stream);
int ma_ce_rows(void* logits, int64_t pitch, const int64_t* targets, int64_t rows, int64_t vocab, int64_t ignore_index,
               float softcap, const float* grad_scale, float* lse, float* nll, int write_grad, int dtype, void* stream);
int ma_ce_loss_reduce(const float* nll, int64_t n, const float* scale, float* loss, void* stream);
int ma_transpose(const void* src, void* dst, int64_t rows, int64_t cols, int src_dtype, int dst_dtype, void* stream);

/* ---- fused QK-RMSNorm + RoPE prologue ------------------------------------------------------------
 * Replaces query_norm/key_norm (model.py:135-172, 366-368) followed by apply_rotary_emb
 * (model.py:97-106, 371-372) with the table gather by position_ids (model.py:744-747):
 *   r = rsqrt(mean(x^2) + eps); y = x*r*(add_unit_offset ? 1+w : w);
 *   out[:D/2] = y[:D/2]*cos - y[D/2:]*sin;  out[D/2:] = y[:D/2]*sin + y[D/2:]*cos   (fp32 math).
 * q_weight/k_weight: fp32 [D] stored parameters, or NULL for no norm (use_qk_norm=False).
 * rope_cos/rope_sin: fp32 [n_pos, D/2].  position_ids: int64 [B,S] contiguous or NULL (= arange).
 * q_rstd/k_rstd: fp32 [B,S,Hq]/[B,S,Hkv] outputs saved for the backward (may be NULL when the
 * matching weight is NULL).  Input and output may alias. */
int ma_prologue_fwd(const ma_tensor4* q_in, const ma_tensor4* k_in, const ma_tensor4* q_out,
                    const ma_tensor4* k_out, const float* q_weight, const float* k_weight,
                    const float* rope_cos, const float* rope_sin, int64_t n_pos,
                    const int64_t* position_ids, float eps, int add_unit_offset, float* q_rstd,
                    float* k_rstd, int dtype, int B, int S, int Hq, int Hkv, int D, void* stream);

/* Backward of the prologue (autograd of the same reference lines).  dq_out/dk_out are the
 * gradients w.r.t. the prologue outputs, dq_in/dk_in receive the gradients w.r.t. its inputs (may
 * alias dq_out/dk_out).  dq_weight/dk_weight: fp32 [D] outputs (NULL with a NULL weight); they are
 * reduced without atomics through `workspace` (ma_prologue_bwd_workspace_bytes). */
size_t ma_prologue_bwd_workspace_bytes(int B, int S, int Hq, int Hkv, int D);
int ma_prologue_bwd(const ma_tensor4* q_in, const ma_tensor4* k_in, const ma_tensor4* dq_out,
                    const ma_tensor4* dk_out, const ma_tensor4* dq_in, const ma_tensor4* dk_in,
                    const float* q_weight, const float* k_weight, const float* rope_cos,
                    const float* rope_sin, int64_t n_pos, const int64_t* position_ids,
                    int add_unit_offset, const float* q_rstd, const float* k_rstd, float* dq_weight,
                    float* dk_weight, void* workspace, size_t workspace_bytes, int dtype, int B,
                    int S, int Hq, int Hkv, int D, void* stream);

/* ---- GQA flash-style attention ---------------------------------------------------------------------
 * Replaces torch.compile(flex_attention)(q, k, v, block_mask, scale, enable_gqa)
 * (model.py:384-396; torch/_higher_order_ops/flex_attention.py:159-267) with the output already in
 * the [B,S,Hq,D] layout that model.py:436-438 produces by a transposed copy.
 *   O = softmax(scale * Q K^T + mask) V, q head h reads kv head h / (Hq/Hkv).
 * lse: fp32 [B,Hq,S] output, natural-log log-sum-exp of the scaled masked scores.
 * map: tile lists from ma_tile_map_build for the SAME (document_ids, causal, window); only tiles in
 * the kv lists are visited, elements of partial tiles are masked with the predicate above.
 * D in {64,128,256}; Hq % Hkv == 0. */
int ma_attn_fwd(const ma_tensor4* q, const ma_tensor4* k, const ma_tensor4* v, const ma_tensor4* out,
                float* lse, const ma_tile_map* map, const int64_t* document_ids, int causal,
                int64_t window, float scale, int dtype, int B, int S, int Hq, int Hkv, int D,
                void* stream);

/* Backward (torch/_higher_order_ops/flex_attention.py:825-993):
 *   delta = rowsum(O * dO); P = exp(S - lse); dV = P^T dO; dS = P * (dO V^T - delta);
 *   dQ = scale * dS K; dK = scale * dS^T Q; dK/dV summed over the Hq/Hkv query heads of a kv head.
 * dK and dV are produced without global atomics (one workgroup owns a kv tile and walks the q-side
 * lists), so results are run-to-run deterministic.
 * workspace: at least ma_attn_bwd_workspace_bytes(...) bytes (holds delta, fp32 [B,Hq,S]).
 * With ma_attn_bwd_ds_workspace_bytes(...) bytes or more (bf16 only; needs map->tile_slot and
 * map->visited_tiles) the dK/dV kernel, which forms dS anyway, also leaves it in the workspace
 * (bf16, one 32 KB slot per VISITED pair of tiles and query head, numbered by map->tile_slot) and
 * the dQ kernel reduces to dQ = scale * dS K instead of recomputing S and dO V^T: the same dK and dV
 * up to the summation order of delta, the same dQ up to the rounding of dS to bf16 (which both
 * variants do before the product), fewer MFMAs, for Hq * visited_tiles * 32 KB (0.45 GB at B=4,
 * S=8192, Hq=8 with documents of some hundred tokens).  Nothing in the workspace needs initialising:
 * inside a slot only the 32 x 32 blocks that hold a visible pair are written, and only those are used. */
size_t ma_attn_bwd_workspace_bytes(int B, int S, int Hq, int Hkv, int D);
size_t ma_attn_bwd_ds_workspace_bytes(int B, int S, int Hq, int64_t visited_tiles);
int ma_attn_bwd(const ma_tensor4* q, const ma_tensor4* k, const ma_tensor4* v, const ma_tensor4* out,
                const ma_tensor4* dout, const float* lse, const ma_tensor4* dq, const ma_tensor4* dk,
                const ma_tensor4* dv, const ma_tile_map* map, const int64_t* document_ids, int causal,
                int64_t window, float scale, void* workspace, size_t workspace_bytes, int dtype,
                int B, int S, int Hq, int Hkv, int D, void* stream);

/* ma_attn_bwd restricted to a subset of its three kernels, for callers that time or overlap them:
 * stages is a bit mask of MA_BWD_DELTA (writes delta into the workspace), MA_BWD_DKV (reads delta,
 * writes dk and dv) and MA_BWD_DQ (reads delta, writes dq).  ma_attn_bwd == all three.  With the
 * larger workspace MA_BWD_DKV also writes dS and MA_BWD_DQ reads it (and no delta): a call with
 * MA_BWD_DQ alone then needs the dS of an earlier MA_BWD_DKV call in the same workspace.  No
 * counterpart in the reference (its backward is one fused Inductor launch,
 * torch/_inductor/kernel/flex/templates/flex_backwards.py.jinja). */
#define MA_BWD_DELTA 1
#define MA_BWD_DKV 2
#define MA_BWD_DQ 4
#define MA_BWD_ALL 7
int ma_attn_bwd_stages(const ma_tensor4* q, const ma_tensor4* k, const ma_tensor4* v, const ma_tensor4* out,
                       const ma_tensor4* dout, const float* lse, const ma_tensor4* dq, const ma_tensor4* dk,
                       const ma_tensor4* dv, const ma_tile_map* map, const int64_t* document_ids, int causal,
                       int64_t window, float scale, void* workspace, size_t workspace_bytes, int dtype,
                       int B, int S, int Hq, int Hkv, int D, int stages, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MAESTER_ATTN_H */
