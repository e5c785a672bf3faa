// bf16 instantiations of the matrix-core conv path (v_mfma_f32_32x32x16_bf16).
#include "mie_conv_mfma_impl.h"

bool mie_launch_conv_mfma(const ConvArgsT<mie_bf16>& a, int k, int s, unsigned cap, hipStream_t st) {
  return launch_any<mie_bf16>(a, k, s, cap, st);
}
bool mie_launch_conv_gates_mfma(const ConvArgsT<mie_bf16>& a, unsigned cap, hipStream_t st) {
  return launch_gates<mie_bf16>(a, cap, st);
}
bool mie_launch_conv_up_mfma(const ConvArgsT<mie_bf16>& a, unsigned cap, hipStream_t st) {
  // 64 -> 32 channels on a large plane: the persistent kernel (mie_upconv_persist.hip)
  return mie_launch_upconv_persist(a, cap, st) || launch_up<mie_bf16>(a, cap, st);
}

#ifdef MIE_WG_PROFILE
// Measurement builds only: the same for the bf16 kernels of this translation unit.
extern "C" __attribute__((visibility("default"))) int mie_set_profile_buffer_bf16(void* p) {
  long long* q = (long long*)p;
  return hipMemcpyToSymbol(HIP_SYMBOL(mie_prof_buf), &q, sizeof(q)) == hipSuccess ? 0 : -4;
}
#endif
