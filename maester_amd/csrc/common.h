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
};

int launch_attn_fwd_f32(const AttnArgs& a, hipStream_t st);
int launch_attn_bwd_f32(const AttnArgs& a, hipStream_t st);
int launch_attn_fwd_bf16(const AttnArgs& a, hipStream_t st);
int launch_attn_bwd_bf16(const AttnArgs& a, hipStream_t st);

inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(MA_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return MA_OK;
}

}  // namespace ma
