// position_ids / document_ids of packed rows, on the device, from the rows' document boundaries.
//
// Counterpart of PackedSFTDataset._generate_position_ids / _generate_document_ids
// (maester/sft/packed_dataset.py:138-185): every boundary i = (start, length) of a row writes
// positions 0, 1, ... and document id i over tokens [start, min(start + length, S)); later
// boundaries overwrite earlier ones; tokens no boundary covers keep position 0 and id -1.
// Per token that is "the last boundary that covers it": one thread per token walks the row's
// boundaries from the last one down (they sit in LDS, a thousand at a time) and stops at the first hit.
#include <hip/hip_runtime.h>

#include "common.h"

namespace ma {

constexpr int kIdsChunk = 1024;

__global__ __launch_bounds__(256) void packed_ids_kernel(const int32_t* __restrict__ starts, const int32_t* __restrict__ lengths,
                                                         const int32_t* __restrict__ counts, int max_docs, int S,
                                                         int64_t* __restrict__ position_ids, int64_t* __restrict__ document_ids) {
    __shared__ int s_start[kIdsChunk], s_end[kIdsChunk];
    const int b = blockIdx.y;
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    const int n = min(max(counts[b], 0), max_docs);
    int doc = -1, pos = 0;
    // chunks of boundaries from the back of the list to its front
    for (int hi = n; hi > 0; hi -= kIdsChunk) {
        const int lo = max(hi - kIdsChunk, 0);
        __syncthreads();
        for (int e = threadIdx.x; e < hi - lo; e += blockDim.x) {
            const int st = starts[(size_t)b * max_docs + lo + e];
            const int len = lengths[(size_t)b * max_docs + lo + e];
            s_start[e] = st;
            s_end[e] = (int)min((int64_t)st + (int64_t)max(len, 0), (int64_t)S);
        }
        __syncthreads();
        if (doc < 0) {
            for (int e = hi - lo - 1; e >= 0; --e) {
                if (t >= s_start[e] && t < s_end[e]) {
                    doc = lo + e;
                    pos = t - s_start[e];
                    break;
                }
            }
        }
    }
    if (t < S) {
        if (position_ids) position_ids[(size_t)b * S + t] = pos;
        if (document_ids) document_ids[(size_t)b * S + t] = doc;
    }
}

int launch_packed_ids(const int32_t* starts, const int32_t* lengths, const int32_t* counts, int B, int max_docs, int S,
                      int64_t* position_ids, int64_t* document_ids, hipStream_t st) {
    hipLaunchKernelGGL(packed_ids_kernel, dim3((S + 255) / 256, B), dim3(256), 0, st, starts, lengths, counts, max_docs, S,
                       position_ids, document_ids);
    return check_launch("packed_ids_kernel");
}

}  // namespace ma
