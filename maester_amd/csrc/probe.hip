// Device probe behind bench.py: what the matrix cores of this GPU sustain on a chain of
// v_mfma_f32_32x32x16_bf16 with nothing else going on -- one wave per SIMD on every compute unit,
// two independent accumulators per wave, operands constant (all ones) or random.  The kernels of the
// library are priced against the published dense peak (2.5 PFLOP/s = 1024 SIMDs x 32768 FLOP / 32
// cycles x 2.4 GHz); this probe records how far the clock itself falls from 2.4 GHz when every SIMD
// issues MFMAs back to back on random data (the chip holds its power limit by lowering the clock),
// i.e. what fraction of that peak any kernel could reach.  No counterpart in the reference.
#include "common.h"
#include "mfma.h"

namespace ma {

__global__ __launch_bounds__(256) void probe_mfma_kernel(int iters, int random_data, unsigned long long* out) {
    f32x16 c0, c1;
#pragma unroll
    for (int v = 0; v < 16; ++v) c0[v] = c1[v] = 0.f;
    bf16x8 a, b;
    unsigned x = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        x = x * 1664525u + 1013904223u;
        a[e] = random_data ? (__bf16)(((int)(x >> 16) % 2001 - 1000) * 0.001f) : (__bf16)1.0f;
        x = x * 1664525u + 1013904223u;
        b[e] = random_data ? (__bf16)(((int)(x >> 16) % 2001 - 1000) * 0.001f) : (__bf16)1.0f;
    }
    const unsigned long long t0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            mfma32_vv(c0, a, b);
            mfma32_vv(c1, a, b);
        }
    }
    mfma_fence();
    mfma_fence();
    const unsigned long long t1 = __builtin_readcyclecounter(), w1 = wall_clock64();
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        out[0] = t1 - t0;                       // shader clocks
        out[1] = w1 - w0;                       // ticks of the constant 100 MHz counter
        out[2] = (unsigned long long)(c0[0] + c1[1] != 12345.f);   // keeps the chains alive
    }
}

int launch_probe_mfma(int iters, int random_data, int workgroups, unsigned long long* out, hipStream_t st) {
    hipLaunchKernelGGL(probe_mfma_kernel, dim3(workgroups), dim3(256), 0, st, iters, random_data, out);
    return check_launch("probe_mfma_kernel");
}

}  // namespace ma
