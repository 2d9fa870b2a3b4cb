// C wrapper around the reference's fused attention forward (both its blocked one-pass routine and
// its plain three-pass one), compiled together with the reference's own src/ops/FlashAttn.cpp where
// it lies; that file needs nothing but include/ppml/FlashAttn.h.  TEST INFRASTRUCTURE ONLY: it lets
// the oracle's restatement be checked against the real reference code.  No reference source is
// copied; the header is included by path at build time.
#include "ppml/FlashAttn.h"

static ppml::FlashAttnConfig config_of(int B, int h, int L, int d, int causal, float scale, float eps, int Bc) {
    ppml::FlashAttnConfig cfg;
    cfg.B = B; cfg.h = h; cfg.L = L; cfg.d = d;
    cfg.causal = causal != 0;
    cfg.scale = scale;
    cfg.softmax_eps = eps;
    if (Bc > 0) cfg.Bc = Bc;
    return cfg;
}

// returns 0 when the reference accepted the arguments, 1 when it refused them
extern "C" int ref_flash_attn_forward(int B, int h, int L, int d, int causal, float scale, float eps, int Bc,
                                      const float* Q, const float* K, const float* V, const float* bias,
                                      float* O, float* LSE) {
    return ppml::flash_attn_forward_cpu(config_of(B, h, L, d, causal, scale, eps, Bc), Q, K, V, bias, O, LSE) ? 0 : 1;
}

extern "C" int ref_flash_attn_forward_plain(int B, int h, int L, int d, int causal, float scale,
                                            const float* Q, const float* K, const float* V, const float* bias,
                                            float* O, float* LSE) {
    return ppml::flash_attn_forward_ref_cpu(config_of(B, h, L, d, causal, scale, 0.0f, 0), Q, K, V, bias, O, LSE) ? 0 : 1;
}

extern "C" int ref_flash_attn_backward(int B, int h, int L, int d, int causal, float scale,
                                       const float* Q, const float* K, const float* V, const float* bias,
                                       const float* O, const float* dO, const float* LSE,
                                       float* dQ, float* dK, float* dV, float* dbias) {
    return ppml::flash_attn_backward_cpu(config_of(B, h, L, d, causal, scale, 0.0f, 0), Q, K, V, bias, O, dO, LSE,
                                         dQ, dK, dV, dbias) ? 0 : 1;
}
