/* CPU restatement of the BlockMask tile lists for the Gemma packed-SFT masks.
 * TEST INFRASTRUCTURE ONLY: loaded by tests and by the bench's checker, never by the product.
 *
 * Follows torch/nn/attention/flex_attention.py (third-party dependency of the reference;
 * call sites maester/models/gemma/model.py:699-706, 723-730):
 *   _convert_mask_to_block_mask (979-1022): per 128x128 tile count of allowed pairs on the
 *       zero-padded mask; full = 16384, partial = 1..16383;
 *   _dense_to_ordered (429-436): set tiles ascending, then unset tiles ascending;
 *   _transpose_ordered (439-441): q-side lists from the transposed tile matrix.
 * Predicate (maester/models/gemma/model.py:203-256):
 *   allowed = same_doc(q,kv) && (!causal || q >= kv) && (window < 0 || (q >= kv && q-kv <= window)).
 */
#include <stdint.h>
#include <stdlib.h>

#define BLK 128

static void ordered(const uint8_t* flag, int T, int stride, int32_t* num, int32_t* idx) {
    int n = 0, p = 0;
    for (int j = 0; j < T; j++) if (flag[(size_t)j * stride]) idx[p++] = j;
    n = p;
    for (int j = 0; j < T; j++) if (!flag[(size_t)j * stride]) idx[p++] = j;
    *num = n;
}

int oracle_tile_map(const int64_t* doc, int B, int S, int causal, long long window,
                    int32_t* kv_num, int32_t* kv_idx, int32_t* fkv_num, int32_t* fkv_idx,
                    int32_t* q_num, int32_t* q_idx, int32_t* fq_num, int32_t* fq_idx) {
    int T = (S + BLK - 1) / BLK;
    uint8_t* part = (uint8_t*)calloc((size_t)T * T, 1);
    uint8_t* full = (uint8_t*)calloc((size_t)T * T, 1);
    if (!part || !full) return -1;
    for (int b = 0; b < B; b++) {
        const int64_t* d = doc ? doc + (size_t)b * S : 0;
        for (int i = 0; i < T; i++) for (int j = 0; j < T; j++) {
            long cnt = 0;
            for (int qi = 0; qi < BLK; qi++) {
                long q = (long)i * BLK + qi;
                if (q >= S) break;
                for (int ki = 0; ki < BLK; ki++) {
                    long kv = (long)j * BLK + ki;
                    if (kv >= S) break;
                    int ok = 1;
                    if (causal && q < kv) ok = 0;
                    if (window >= 0 && !(q >= kv && q - kv <= window)) ok = 0;
                    if (d && d[q] != d[kv]) ok = 0;
                    cnt += ok;
                }
            }
            part[(size_t)i * T + j] = (cnt > 0 && cnt < BLK * BLK);
            full[(size_t)i * T + j] = (cnt == BLK * BLK);
        }
        for (int i = 0; i < T; i++) {
            size_t r = (size_t)b * T + i;
            ordered(part + (size_t)i * T, T, 1, kv_num + r, kv_idx + r * T);
            ordered(full + (size_t)i * T, T, 1, fkv_num + r, fkv_idx + r * T);
            ordered(part + i, T, T, q_num + r, q_idx + r * T);
            ordered(full + i, T, T, fq_num + r, fq_idx + r * T);
        }
    }
    free(part); free(full);
    return 0;
}
