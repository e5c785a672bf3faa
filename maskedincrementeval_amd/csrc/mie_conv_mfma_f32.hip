// fp32 instantiations of the matrix-core conv path (v_mfma_f32_32x32x2_f32) and the shape predicate.
#include "mie_conv_mfma_impl.h"

// Whether some kernel variant takes the shape: whole staging chunks of input channels (stride 2
// may fall back to the half depth) and whole output slabs for the wave splits that depth allows.
bool mie_conv_mfma_takes(int k, int s, int dtype, int c1, int c2, int cout) {
  const int mult = dtype == MIE_DTYPE_BF16 ? 2 : 1;
  for (int half = 0; half < (s == 2 ? 2 : 1); ++half) {
    const int cc = stage_channels(k, s, half != 0), depth = cc * mult, nq = cc / 8;
    const int cmul = nq >= 4 ? 32 : (nq >= 2 ? 64 : 128);
    if (c1 % depth == 0 && c2 % depth == 0 && cout % cmul == 0) return true;
  }
  return false;
}

bool mie_conv_x3_takes(int k, int s, int c1, int c2, int cout) { return x3_takes(k, s, c1, c2, cout); }

bool mie_launch_conv_mfma(const ConvArgsT<float>& a, int k, int s, unsigned cap, hipStream_t st) {
  return launch_any<float>(a, k, s, cap, st);
}
bool mie_launch_conv_gates_mfma(const ConvArgsT<float>& a, unsigned cap, hipStream_t st) {
  return launch_gates<float>(a, cap, st);
}
bool mie_launch_conv_up_mfma(const ConvArgsT<float>& a, unsigned cap, hipStream_t st) {
  return launch_up<float>(a, cap, st);
}

#ifdef MIE_WG_PROFILE
// Measurement builds only: where the fp32 kernels of this translation unit write their workgroup timelines
// (NULL switches the stamps off).  The buffer needs 128 bytes per workgroup of the launches it covers.
extern "C" __attribute__((visibility("default"))) int mie_set_profile_buffer(void* p) {
  long long* q = (long long*)p;
  return hipMemcpyToSymbol(HIP_SYMBOL(mie_prof_buf), &q, sizeof(q)) == hipSuccess ? 0 : -4;
}
#endif
