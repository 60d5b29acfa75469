#include "common.h"
namespace ma {
int launch_attn_bwd_bf16(const AttnArgs& a, hipStream_t st) {
    (void)a; (void)st;
    return fail(MA_ERR_UNSUPPORTED, "attn_bwd bf16: not built yet");
}
}
