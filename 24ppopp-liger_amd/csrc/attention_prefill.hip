// attention_prefill.hip -- fused LDS-tiled prefill attention (placeholder until the kernel lands).
#include "common.cuh"

using namespace lg;

extern "C" int lg_attn_prefill_f16(const void* q_buf, const void* k_buf, const void* v_buf, const void* attr_mask,
                                   void* out, int batch, int seq, int head_num, int size_per_head, float scalar,
                                   int causal, int out_layout, void* stream) {
    (void)q_buf; (void)k_buf; (void)v_buf; (void)attr_mask; (void)out; (void)batch; (void)seq; (void)head_num;
    (void)size_per_head; (void)scalar; (void)causal; (void)out_layout; (void)stream;
    set_error("attn_prefill: not available in this build");
    return LG_ERR_INVALID;
}
