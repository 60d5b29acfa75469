// C-ABI layer: argument validation (runs on the host before any launch, so every error path is
// reachable without a GPU) and dispatch to the kernel launchers.  See include/maester_attn.h.
#include "common.h"

#include <string.h>

namespace ma {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

static int check_dims(const char* who, int B, int S, int Hq, int Hkv, int D) {
    if (B <= 0 || S <= 0) return fail(MA_ERR_BAD_ARG, "%s: B=%d and S=%d must be positive", who, B, S);
    if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0)
        return fail(MA_ERR_BAD_ARG, "%s: Hq=%d must be a positive multiple of Hkv=%d", who, Hq, Hkv);
    if (B > 65535 || Hq > 65535) return fail(MA_ERR_BAD_ARG, "%s: B=%d / Hq=%d exceed the grid limit 65535", who, B, Hq);
    if ((int64_t)B * S > (int64_t)1 << 30) return fail(MA_ERR_BAD_ARG, "%s: B*S=%lld too large", who, (long long)B * S);
    if (D != 64 && D != 128 && D != 256) return fail(MA_ERR_UNSUPPORTED, "%s: head_dim %d not in {64,128,256}", who, D);
    // the attention kernels keep a step as one word: 24 bits of row number, 5 bits of query head within its group
    if (S >= (1 << 24)) return fail(MA_ERR_UNSUPPORTED, "%s: S=%d is 2^24 or more", who, S);
    if (Hq / Hkv > 32) return fail(MA_ERR_UNSUPPORTED, "%s: %d query heads per kv head (at most 32)", who, Hq / Hkv);
    return MA_OK;
}

static int check_dtype(const char* who, int dtype) {
    if (dtype != MA_DTYPE_F32 && dtype != MA_DTYPE_BF16)
        return fail(MA_ERR_BAD_ARG, "%s: dtype %d is neither MA_DTYPE_F32 nor MA_DTYPE_BF16", who, dtype);
    return MA_OK;
}

static int check_tensor(const char* who, const char* name, const ma_tensor4* t, int dtype) {
    if (!t || !t->ptr) return fail(MA_ERR_BAD_ARG, "%s: tensor %s is NULL", who, name);
    const int elt = dtype == MA_DTYPE_BF16 ? 2 : 4;
    // rows are moved with 16-byte vector accesses
    const int64_t al = 16 / elt;
    if (((uintptr_t)t->ptr & 15) != 0) return fail(MA_ERR_BAD_ARG, "%s: %s is not 16-byte aligned", who, name);
    if (t->stride_b % al || t->stride_s % al || t->stride_h % al)
        return fail(MA_ERR_BAD_ARG, "%s: strides of %s (%lld,%lld,%lld) must be multiples of %lld elements", who, name,
                    (long long)t->stride_b, (long long)t->stride_s, (long long)t->stride_h, (long long)al);
    if (t->stride_b < 0 || t->stride_s <= 0 || t->stride_h < 0)
        return fail(MA_ERR_BAD_ARG, "%s: strides of %s must be non-negative (stride_s positive)", who, name);
    // the kernels address the rows of a 128-row tile with 32-bit byte offsets
    if (t->stride_s * elt >= ((int64_t)1 << 24))
        return fail(MA_ERR_UNSUPPORTED, "%s: row stride of %s (%lld elements) is 16 MiB or more", who, name, (long long)t->stride_s);
    return MA_OK;
}

static int check_map(const char* who, const ma_tile_map* m, bool need_kv, bool need_q) {
    if (!m) return fail(MA_ERR_BAD_ARG, "%s: tile map is NULL", who);
    if (need_kv && (!m->kv_num_blocks || !m->kv_indices || !m->full_kv_num_blocks || !m->full_kv_indices))
        return fail(MA_ERR_BAD_ARG, "%s: tile map lacks the kv-side lists", who);
    if (need_q && (!m->q_num_blocks || !m->q_indices || !m->full_q_num_blocks || !m->full_q_indices))
        return fail(MA_ERR_BAD_ARG, "%s: tile map lacks the q-side lists", who);
    return MA_OK;
}

static int check_mask(const char* who, int causal, int64_t window) {
    if (causal != 0 && causal != 1) return fail(MA_ERR_BAD_ARG, "%s: causal must be 0 or 1, got %d", who, causal);
    if (window < -1) return fail(MA_ERR_BAD_ARG, "%s: window must be -1 (none) or >= 0, got %lld", who, (long long)window);
    return MA_OK;
}

}  // namespace ma

using namespace ma;

#define MA_TRY(expr)            \
    do {                        \
        int rc__ = (expr);      \
        if (rc__) return rc__;  \
    } while (0)

extern "C" {

int ma_version(void) { return MA_ABI_VERSION; }

const char* ma_last_error(void) { return g_err; }

int ma_probe_mfma(int iters, int random_data, int workgroups, uint64_t* out, void* stream) {
    const char* who = "ma_probe_mfma";
    if (iters <= 0 || iters > (1 << 20)) return fail(MA_ERR_BAD_ARG, "%s: iters=%d out of range (1 .. 2^20)", who, iters);
    if (workgroups <= 0 || workgroups > 65535) return fail(MA_ERR_BAD_ARG, "%s: workgroups=%d out of range", who, workgroups);
    if (!out || ((uintptr_t)out & 7) != 0) return fail(MA_ERR_BAD_ARG, "%s: out is NULL or not 8-byte aligned", who);
    return launch_probe_mfma(iters, random_data ? 1 : 0, workgroups, (unsigned long long*)out, (hipStream_t)stream);
}

size_t ma_tile_map_workspace_bytes(int B, int S) {
    if (B <= 0 || S <= 0) return 0;
    const size_t T = ((size_t)S + MA_TILE - 1) / MA_TILE;
    // class byte per tile (rounded up to 16 bytes) | (min, max) document id per tile | counter | list of
    // the tiles that need an exact count
    return (((size_t)B * T * T + 15) & ~(size_t)15) + (size_t)B * T * 2 * sizeof(int64_t) + 16 + (size_t)B * T * T * sizeof(int32_t);
}

static int check_tile_map_args(const char* who, int B, int S, int causal, int64_t window, const ma_tile_map* out) {
    if (B <= 0 || S <= 0) return fail(MA_ERR_BAD_ARG, "%s: B=%d and S=%d must be positive", who, B, S);
    if (B > 65535) return fail(MA_ERR_BAD_ARG, "%s: B=%d exceeds the grid limit 65535", who, B);
    const int64_t T = ((int64_t)S + MA_TILE - 1) / MA_TILE;
    if (T > 65535) return fail(MA_ERR_BAD_ARG, "%s: S=%d gives %lld tiles per side, limit 65535", who, S, (long long)T);
    // tiles are numbered b*T*T + i*T + j in 32 bits (the list of tiles that need an exact count)
    if ((int64_t)B * T * T >= ((int64_t)1 << 31))
        return fail(MA_ERR_UNSUPPORTED, "%s: B=%d, S=%d gives %lld tiles, limit 2^31", who, B, S, (long long)((int64_t)B * T * T));
    MA_TRY(check_mask(who, causal, window));
    MA_TRY(check_map(who, out, true, true));
    return MA_OK;
}

int ma_tile_map_build(const int64_t* document_ids, int B, int S, int causal, int64_t window, const ma_tile_map* out,
                      void* workspace, size_t workspace_bytes, void* stream) {
    const char* who = "ma_tile_map_build";
    MA_TRY(check_tile_map_args(who, B, S, causal, window, out));
    if (!workspace || workspace_bytes < ma_tile_map_workspace_bytes(B, S))
        return fail(MA_ERR_BAD_ARG, "%s: workspace of %zu bytes, need %zu", who, workspace ? workspace_bytes : (size_t)0,
                    ma_tile_map_workspace_bytes(B, S));
    return launch_tile_map(document_ids, B, S, causal, window, *out, workspace, (hipStream_t)stream);
}

int ma_tile_map_build_static(const int64_t* document_ids, int B, int S, int causal, int64_t window, const ma_tile_map* out,
                             void* stream) {
    const char* who = "ma_tile_map_build_static";
    MA_TRY(check_tile_map_args(who, B, S, causal, window, out));
    const size_t need = ma_tile_map_workspace_bytes(B, S);
    if (need > (size_t)MA_TILE_MAP_STATIC_BYTES)
        return fail(MA_ERR_UNSUPPORTED, "%s: B=%d, S=%d needs %zu bytes of scratch, the library holds %zu; use ma_tile_map_build with a workspace",
                    who, B, S, need, (size_t)MA_TILE_MAP_STATIC_BYTES);
    void* ws = nullptr;
    MA_TRY(static_tile_map_scratch(&ws));
    return launch_tile_map(document_ids, B, S, causal, window, *out, ws, (hipStream_t)stream);
}

static int check_norm(const char* who, const void* x, const float* weight, int64_t rows, int dim, int dtype) {
    MA_TRY(check_dtype(who, dtype));
    if (rows <= 0 || rows > ((int64_t)1 << 31) - 1) return fail(MA_ERR_BAD_ARG, "%s: rows=%lld out of range", who, (long long)rows);
    if (dim <= 0 || dim % 8 != 0 || dim > 8192)
        return fail(MA_ERR_UNSUPPORTED, "%s: dim=%d must be a multiple of 8, at most 8192", who, dim);
    if (!x || !weight) return fail(MA_ERR_BAD_ARG, "%s: x / weight is NULL", who);
    if (((uintptr_t)x & 15) != 0 || ((uintptr_t)weight & 15) != 0) return fail(MA_ERR_BAD_ARG, "%s: x / weight not 16-byte aligned", who);
    return MA_OK;
}

size_t ma_rmsnorm_bwd_workspace_bytes(int64_t rows, int dim) {
    if (rows <= 0 || dim <= 0) return 0;
    return (size_t)rmsnorm_bwd_blocks(rows) * dim * sizeof(float);
}

int ma_rmsnorm_fwd(const void* x, const void* residual, const float* weight, void* out, float* rstd, int64_t rows, int dim,
                   float eps, int add_unit_offset, int dtype, void* stream) {
    const char* who = "ma_rmsnorm_fwd";
    MA_TRY(check_norm(who, x, weight, rows, dim, dtype));
    if (!out || ((uintptr_t)out & 15) != 0) return fail(MA_ERR_BAD_ARG, "%s: out is NULL or not 16-byte aligned", who);
    if (residual && ((uintptr_t)residual & 15) != 0) return fail(MA_ERR_BAD_ARG, "%s: residual not 16-byte aligned", who);
    if (!(eps >= 0.f)) return fail(MA_ERR_BAD_ARG, "%s: eps must be >= 0", who);
    return launch_rmsnorm_fwd(x, residual, weight, out, rstd, rows, dim, eps, add_unit_offset ? 1 : 0, dtype, (hipStream_t)stream);
}

int ma_rmsnorm_bwd(const void* x, const float* weight, const float* rstd, const void* dout, void* dx, float* dweight,
                   void* workspace, size_t workspace_bytes, int64_t rows, int dim, int add_unit_offset, int dtype, void* stream) {
    const char* who = "ma_rmsnorm_bwd";
    MA_TRY(check_norm(who, x, weight, rows, dim, dtype));
    if (!rstd || !dout || !dx || !dweight) return fail(MA_ERR_BAD_ARG, "%s: rstd / dout / dx / dweight is NULL", who);
    if ((((uintptr_t)dout | (uintptr_t)dx) & 15) != 0) return fail(MA_ERR_BAD_ARG, "%s: dout / dx not 16-byte aligned", who);
    if (!workspace || workspace_bytes < ma_rmsnorm_bwd_workspace_bytes(rows, dim))
        return fail(MA_ERR_BAD_ARG, "%s: workspace of %zu bytes, need %zu", who, workspace ? workspace_bytes : (size_t)0,
                    ma_rmsnorm_bwd_workspace_bytes(rows, dim));
    return launch_rmsnorm_bwd(x, weight, rstd, dout, dx, dweight, workspace, rows, dim, add_unit_offset ? 1 : 0, dtype,
                              (hipStream_t)stream);
}

int ma_ce_valid_count(const int64_t* targets, int64_t n, int64_t ignore_index, int64_t vocab, float* stats, void* stream) {
    const char* who = "ma_ce_valid_count";
    if (!targets || !stats) return fail(MA_ERR_BAD_ARG, "%s: targets / stats is NULL", who);
    if (n <= 0) return fail(MA_ERR_BAD_ARG, "%s: n=%lld must be positive", who, (long long)n);
    if (vocab <= 0 || vocab > ((int64_t)1 << 31) - 1) return fail(MA_ERR_BAD_ARG, "%s: vocab=%lld out of range", who, (long long)vocab);
    return launch_ce_valid_count(targets, n, ignore_index, (int)vocab, stats, (hipStream_t)stream);
}

int ma_ce_rows(void* logits, int64_t pitch, const int64_t* targets, int64_t rows, int64_t vocab, int64_t ignore_index,
               float softcap, const float* grad_scale, float* lse, float* nll, int write_grad, int dtype, void* stream) {
    const char* who = "ma_ce_rows";
    MA_TRY(check_dtype(who, dtype));
    if (!logits || !targets) return fail(MA_ERR_BAD_ARG, "%s: logits / targets is NULL", who);
    if (rows <= 0 || rows > ((int64_t)1 << 31) - 1) return fail(MA_ERR_BAD_ARG, "%s: rows=%lld out of range", who, (long long)rows);
    if (vocab <= 0 || vocab > ((int64_t)1 << 31) - 1) return fail(MA_ERR_BAD_ARG, "%s: vocab=%lld out of range", who, (long long)vocab);
    if (pitch < vocab) return fail(MA_ERR_BAD_ARG, "%s: pitch=%lld is below vocab=%lld", who, (long long)pitch, (long long)vocab);
    if (!(softcap >= 0.f)) return fail(MA_ERR_BAD_ARG, "%s: softcap must be >= 0 (0 = none)", who);
    const int elt = dtype == MA_DTYPE_BF16 ? 2 : 4;
    if (((uintptr_t)logits & (elt - 1)) != 0) return fail(MA_ERR_BAD_ARG, "%s: logits not aligned to its element size", who);
    return launch_ce_rows(logits, pitch, targets, rows, (int)vocab, ignore_index, softcap, grad_scale, lse, nll, write_grad ? 1 : 0,
                          dtype, (hipStream_t)stream);
}

int ma_transpose(const void* src, void* dst, int64_t rows, int64_t cols, int src_dtype, int dst_dtype, void* stream) {
    const char* who = "ma_transpose";
    MA_TRY(check_dtype(who, src_dtype));
    MA_TRY(check_dtype(who, dst_dtype));
    if (src_dtype == MA_DTYPE_BF16 && dst_dtype != MA_DTYPE_BF16)
        return fail(MA_ERR_UNSUPPORTED, "%s: bf16 -> fp32 is not offered (same dtype, or fp32 -> bf16)", who);
    if (!src || !dst || src == dst) return fail(MA_ERR_BAD_ARG, "%s: src / dst is NULL, or the same buffer", who);
    if (rows <= 0 || cols <= 0) return fail(MA_ERR_BAD_ARG, "%s: rows=%lld, cols=%lld must be positive", who, (long long)rows, (long long)cols);
    if ((rows + 63) / 64 > 65535) return fail(MA_ERR_UNSUPPORTED, "%s: rows=%lld exceeds 65535 tiles of 64", who, (long long)rows);
    return launch_transpose(src, dst, rows, cols, src_dtype, dst_dtype, (hipStream_t)stream);
}

int ma_ce_loss_reduce(const float* nll, int64_t n, const float* scale, float* loss, void* stream) {
    const char* who = "ma_ce_loss_reduce";
    if (!nll || !loss) return fail(MA_ERR_BAD_ARG, "%s: nll / loss is NULL", who);
    if (n <= 0) return fail(MA_ERR_BAD_ARG, "%s: n=%lld must be positive", who, (long long)n);
    return launch_ce_loss_reduce(nll, n, scale, loss, (hipStream_t)stream);
}

int ma_packed_ids_build(const int32_t* starts, const int32_t* lengths, const int32_t* counts, int B, int max_docs, int S,
                        int64_t* position_ids, int64_t* document_ids, void* stream) {
    const char* who = "ma_packed_ids_build";
    if (B <= 0 || S <= 0) return fail(MA_ERR_BAD_ARG, "%s: B=%d and S=%d must be positive", who, B, S);
    if (B > 65535) return fail(MA_ERR_BAD_ARG, "%s: B=%d exceeds the grid limit 65535", who, B);
    if (max_docs < 0) return fail(MA_ERR_BAD_ARG, "%s: max_docs=%d is negative", who, max_docs);
    if (!counts) return fail(MA_ERR_BAD_ARG, "%s: counts is NULL", who);
    if (max_docs > 0 && (!starts || !lengths)) return fail(MA_ERR_BAD_ARG, "%s: starts / lengths are NULL", who);
    if (!position_ids && !document_ids) return fail(MA_ERR_BAD_ARG, "%s: both outputs are NULL", who);
    return launch_packed_ids(starts, lengths, counts, B, max_docs, S, position_ids, document_ids, (hipStream_t)stream);
}

int ma_prologue_fwd(const ma_tensor4* q_in, const ma_tensor4* k_in, const ma_tensor4* q_out, const ma_tensor4* k_out,
                    const float* q_weight, const float* k_weight, const float* rope_cos, const float* rope_sin,
                    int64_t n_pos, const int64_t* position_ids, float eps, int add_unit_offset, float* q_rstd,
                    float* k_rstd, int dtype, int B, int S, int Hq, int Hkv, int D, void* stream) {
    const char* who = "ma_prologue_fwd";
    MA_TRY(check_dims(who, B, S, Hq, Hkv, D));
    MA_TRY(check_dtype(who, dtype));
    MA_TRY(check_tensor(who, "q_in", q_in, dtype));
    MA_TRY(check_tensor(who, "k_in", k_in, dtype));
    MA_TRY(check_tensor(who, "q_out", q_out, dtype));
    MA_TRY(check_tensor(who, "k_out", k_out, dtype));
    if (!rope_cos || !rope_sin) return fail(MA_ERR_BAD_ARG, "%s: rope tables are NULL", who);
    if (n_pos <= 0) return fail(MA_ERR_BAD_ARG, "%s: n_pos=%lld must be positive", who, (long long)n_pos);
    if (!position_ids && n_pos < S)
        return fail(MA_ERR_BAD_ARG, "%s: default positions need n_pos >= S (%lld < %d)", who, (long long)n_pos, S);
    if (q_weight && !q_rstd) return fail(MA_ERR_BAD_ARG, "%s: q_rstd is NULL but q_weight is given", who);
    if (k_weight && !k_rstd) return fail(MA_ERR_BAD_ARG, "%s: k_rstd is NULL but k_weight is given", who);
    if (!(eps >= 0.f)) return fail(MA_ERR_BAD_ARG, "%s: eps must be >= 0", who);
    return launch_prologue_fwd(*q_in, *k_in, *q_out, *k_out, q_weight, k_weight, rope_cos, rope_sin, n_pos,
                               position_ids, eps, add_unit_offset ? 1 : 0, q_rstd, k_rstd, dtype, B, S, Hq, Hkv, D,
                               (hipStream_t)stream);
}

size_t ma_prologue_bwd_workspace_bytes(int B, int S, int Hq, int Hkv, int D) {
    (void)Hq; (void)Hkv;
    if (B <= 0 || S <= 0 || D <= 0) return 0;
    return (size_t)prologue_bwd_blocks(B, S) * 2 * (size_t)D * sizeof(float);
}

int ma_prologue_bwd(const ma_tensor4* q_in, const ma_tensor4* k_in, const ma_tensor4* dq_out, const ma_tensor4* dk_out,
                    const ma_tensor4* dq_in, const ma_tensor4* dk_in, const float* q_weight, const float* k_weight,
                    const float* rope_cos, const float* rope_sin, int64_t n_pos, const int64_t* position_ids,
                    int add_unit_offset, const float* q_rstd, const float* k_rstd, float* dq_weight, float* dk_weight,
                    void* workspace, size_t workspace_bytes, int dtype, int B, int S, int Hq, int Hkv, int D,
                    void* stream) {
    const char* who = "ma_prologue_bwd";
    MA_TRY(check_dims(who, B, S, Hq, Hkv, D));
    MA_TRY(check_dtype(who, dtype));
    MA_TRY(check_tensor(who, "dq_out", dq_out, dtype));
    MA_TRY(check_tensor(who, "dk_out", dk_out, dtype));
    MA_TRY(check_tensor(who, "dq_in", dq_in, dtype));
    MA_TRY(check_tensor(who, "dk_in", dk_in, dtype));
    if (q_weight) MA_TRY(check_tensor(who, "q_in", q_in, dtype));
    if (k_weight) MA_TRY(check_tensor(who, "k_in", k_in, dtype));
    if (!rope_cos || !rope_sin) return fail(MA_ERR_BAD_ARG, "%s: rope tables are NULL", who);
    if (n_pos <= 0) return fail(MA_ERR_BAD_ARG, "%s: n_pos=%lld must be positive", who, (long long)n_pos);
    if (!position_ids && n_pos < S)
        return fail(MA_ERR_BAD_ARG, "%s: default positions need n_pos >= S (%lld < %d)", who, (long long)n_pos, S);
    if (q_weight && (!q_rstd || !dq_weight)) return fail(MA_ERR_BAD_ARG, "%s: q_weight needs q_rstd and dq_weight", who);
    if (k_weight && (!k_rstd || !dk_weight)) return fail(MA_ERR_BAD_ARG, "%s: k_weight needs k_rstd and dk_weight", who);
    if ((q_weight || k_weight) &&
        (!workspace || workspace_bytes < ma_prologue_bwd_workspace_bytes(B, S, Hq, Hkv, D)))
        return fail(MA_ERR_BAD_ARG, "%s: workspace of %zu bytes, need %zu", who, workspace ? workspace_bytes : (size_t)0,
                    ma_prologue_bwd_workspace_bytes(B, S, Hq, Hkv, D));
    ma_tensor4 none = {nullptr, 0, 0, 0};
    return launch_prologue_bwd(q_in ? *q_in : none, k_in ? *k_in : none, *dq_out, *dk_out, *dq_in, *dk_in, q_weight,
                               k_weight, rope_cos, rope_sin, n_pos, position_ids, add_unit_offset ? 1 : 0, q_rstd,
                               k_rstd, dq_weight, dk_weight, workspace, dtype, B, S, Hq, Hkv, D, (hipStream_t)stream);
}

static int fill_attn(const char* who, AttnArgs& a, const ma_tensor4* q, const ma_tensor4* k, const ma_tensor4* v,
                     const ma_tensor4* out, const ma_tile_map* map, const int64_t* document_ids, int causal,
                     int64_t window, float scale, int dtype, int B, int S, int Hq, int Hkv, int D, bool bwd) {
    a.ds = nullptr;
    MA_TRY(check_dims(who, B, S, Hq, Hkv, D));
    MA_TRY(check_dtype(who, dtype));
    MA_TRY(check_tensor(who, "q", q, dtype));
    MA_TRY(check_tensor(who, "k", k, dtype));
    MA_TRY(check_tensor(who, "v", v, dtype));
    MA_TRY(check_tensor(who, "out", out, dtype));
    MA_TRY(check_mask(who, causal, window));
    MA_TRY(check_map(who, map, true, bwd));
    if (!(scale > 0.f) || scale != scale) return fail(MA_ERR_BAD_ARG, "%s: scale must be positive and finite", who);
    memset(&a, 0, sizeof(a));
    a.q = *q; a.k = *k; a.v = *v; a.o = *out;
    a.map = *map;
    a.doc = document_ids;
    a.causal = causal;
    a.window = window;
    a.scale = scale;
    a.B = B; a.S = S; a.Hq = Hq; a.Hkv = Hkv; a.D = D;
    a.T = (S + MA_TILE - 1) / MA_TILE;
    return MA_OK;
}

int ma_attn_fwd(const ma_tensor4* q, const ma_tensor4* k, const ma_tensor4* v, const ma_tensor4* out, float* lse,
                const ma_tile_map* map, const int64_t* document_ids, int causal, int64_t window, float scale, int dtype,
                int B, int S, int Hq, int Hkv, int D, void* stream) {
    const char* who = "ma_attn_fwd";
    AttnArgs a;
    MA_TRY(fill_attn(who, a, q, k, v, out, map, document_ids, causal, window, scale, dtype, B, S, Hq, Hkv, D, false));
    if (!lse) return fail(MA_ERR_BAD_ARG, "%s: lse is NULL", who);
    a.lse = lse;
    return dtype == MA_DTYPE_BF16 ? launch_attn_fwd_bf16(a, (hipStream_t)stream)
                                  : launch_attn_fwd_f32(a, (hipStream_t)stream);
}

size_t ma_attn_bwd_workspace_bytes(int B, int S, int Hq, int Hkv, int D) {
    (void)Hkv; (void)D;
    if (B <= 0 || S <= 0 || Hq <= 0) return 0;
    return (size_t)B * Hq * S * sizeof(float);  // delta
}

static size_t delta_bytes_aligned(int B, int S, int Hq) { return (((size_t)B * Hq * S * sizeof(float)) + 255) & ~(size_t)255; }

size_t ma_attn_bwd_ds_workspace_bytes(int B, int S, int Hq, int64_t visited_tiles) {
    if (B <= 0 || S <= 0 || Hq <= 0 || visited_tiles <= 0) return 0;
    return delta_bytes_aligned(B, S, Hq) + (size_t)Hq * (size_t)visited_tiles * MA_TILE * MA_TILE * 2;  // delta, then dS^T in bf16
}

int ma_attn_bwd(const ma_tensor4* q, const ma_tensor4* k, const ma_tensor4* v, const ma_tensor4* out,
                const ma_tensor4* dout, const float* lse, const ma_tensor4* dq, const ma_tensor4* dk,
                const ma_tensor4* dv, const ma_tile_map* map, const int64_t* document_ids, int causal, int64_t window,
                float scale, void* workspace, size_t workspace_bytes, int dtype, int B, int S, int Hq, int Hkv, int D,
                void* stream) {
    return ma_attn_bwd_stages(q, k, v, out, dout, lse, dq, dk, dv, map, document_ids, causal, window, scale, workspace,
                              workspace_bytes, dtype, B, S, Hq, Hkv, D, MA_BWD_ALL, stream);
}

int ma_attn_bwd_stages(const ma_tensor4* q, const ma_tensor4* k, const ma_tensor4* v, const ma_tensor4* out,
                       const ma_tensor4* dout, const float* lse, const ma_tensor4* dq, const ma_tensor4* dk,
                       const ma_tensor4* dv, const ma_tile_map* map, const int64_t* document_ids, int causal,
                       int64_t window, float scale, void* workspace, size_t workspace_bytes, int dtype, int B, int S,
                       int Hq, int Hkv, int D, int stages, void* stream) {
    const char* who = "ma_attn_bwd";
    if (stages <= 0 || (stages & ~MA_BWD_ALL)) return fail(MA_ERR_BAD_ARG, "%s: stages mask %d is invalid", who, stages);
    AttnArgs a;
    MA_TRY(fill_attn(who, a, q, k, v, out, map, document_ids, causal, window, scale, dtype, B, S, Hq, Hkv, D, true));
    MA_TRY(check_tensor(who, "dout", dout, dtype));
    MA_TRY(check_tensor(who, "dq", dq, dtype));
    MA_TRY(check_tensor(who, "dk", dk, dtype));
    MA_TRY(check_tensor(who, "dv", dv, dtype));
    if (!lse) return fail(MA_ERR_BAD_ARG, "%s: lse is NULL", who);
    if (!workspace || workspace_bytes < ma_attn_bwd_workspace_bytes(B, S, Hq, Hkv, D))
        return fail(MA_ERR_BAD_ARG, "%s: workspace of %zu bytes, need %zu", who, workspace ? workspace_bytes : (size_t)0,
                    ma_attn_bwd_workspace_bytes(B, S, Hq, Hkv, D));
    if (((uintptr_t)workspace & 15) != 0) return fail(MA_ERR_BAD_ARG, "%s: workspace is not 16-byte aligned", who);
    a.dout = *dout; a.dq = *dq; a.dk = *dk; a.dv = *dv;
    a.lse = (float*)lse;
    a.delta = (float*)workspace;
    a.stages = stages;
    // a workspace large enough for the dS^T of every visited tile selects the hand-over between the two bf16 kernels
    const int64_t T64 = ((int64_t)S + MA_TILE - 1) / MA_TILE;
    if (dtype == MA_DTYPE_BF16 && map->tile_slot && map->visited_tiles > 0 && map->visited_tiles <= (int64_t)B * T64 * T64 &&
        workspace_bytes >= ma_attn_bwd_ds_workspace_bytes(B, S, Hq, map->visited_tiles)) {
        a.ds = (char*)workspace + delta_bytes_aligned(B, S, Hq);
        a.ds_tiles = map->visited_tiles;
    }
    return dtype == MA_DTYPE_BF16 ? launch_attn_bwd_bf16(a, (hipStream_t)stream)
                                  : launch_attn_bwd_f32(a, (hipStream_t)stream);
}

}  // extern "C"
