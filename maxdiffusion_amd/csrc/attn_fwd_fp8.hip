// fp8-e4m3 attention forward (placeholder until the MFMA kernel lands).
#include "mdattn_common.h"

extern "C" int mdattn_fwd_fp8(void* stream, const void* q8, const void* k8, const void* v8, void* out, float* lse,
                              int B, int H, int Sq, int Skv, int D,
                              const mdattn_strides* q_strides, const mdattn_strides* k_strides,
                              const mdattn_strides* v_strides, const mdattn_strides* o_strides, float scale,
                              const float* q_scale, const float* k_scale, const float* v_scale) {
  (void)stream; (void)q8; (void)k8; (void)v8; (void)out; (void)lse; (void)B; (void)H; (void)Sq; (void)Skv; (void)D;
  (void)q_strides; (void)k_strides; (void)v_strides; (void)o_strides; (void)scale; (void)q_scale; (void)k_scale; (void)v_scale;
  return MDATTN_E_UNSUPPORTED;
}
