// bf16 instantiations of the matrix-core conv path (v_mfma_f32_32x32x16_bf16).
#include "mie_conv_mfma_impl.h"

bool mie_launch_conv_mfma(const ConvArgsT<mie_bf16>& a, int k, int s, unsigned cap, hipStream_t st) {
  return launch_any<mie_bf16>(a, k, s, cap, st);
}
bool mie_launch_conv_gates_mfma(const ConvArgsT<mie_bf16>& a, unsigned cap, hipStream_t st) {
  return launch_gates<mie_bf16>(a, cap, st);
}
bool mie_launch_conv_up_mfma(const ConvArgsT<mie_bf16>& a, unsigned cap, hipStream_t st) {
  return launch_up<mie_bf16>(a, cap, st);
}
