// Masked conv on the matrix cores for layers with very few input channels: the network heads (5 or 4
// event bins -> 32 / 64 channels, 5x5 or 3x3).  Their contraction, K*K*Cin = 36 .. 125, is too short for
// the staged implicit GEMM of mie_conv_mfma_impl.h (whole chunks of 32 channels, 16-byte channel slots),
// and on the VALU path they run at a tenth of the vector peak.  Here the whole problem of a workgroup
// fits LDS at once:
//   * one 256-thread workgroup = one active 8x8 output tile x 32 output channels;
//   * the input tile plus halo is staged in fp32, channels padded to 8 (pixel stride 9 floats), inactive
//     pixels zero-filled without being read; bf16 deltas are widened while staging, so one kernel body
//     (v_mfma_f32_32x32x2_f32) serves both element types -- products of bf16 values are exact in fp32;
//   * the filter slab [tap][8 channels][32 columns] is staged from the plain fp32 filter, zero rows for
//     the padding channels;
//   * k = (tap, channel pair); wave w multiplies the 32-pixel block w & 1 (tile rows 0-3 / 4-7) for the
//     taps of parity w >> 1, only the ceil(Cin / 2) channel pairs that exist; the two tap halves meet in
//     LDS and are added in a fixed order; epilogue as everywhere (addend, reservoir, activation, refresh).
// One input only (x2 unsupported), stride 1 or 2, K = 3 or 5, Cout % 32 == 0.
// UP: the input is up2x(x), the bilinear x2 up-sampling of a delta given at half resolution (a.h_in / a.w_in are
// the up-sampled size): every staged pixel is blended from its four source pixels while staging, the up-sampled
// tensor is never formed (the 2-channel flow estimate in front of an EVFlowNet decoder).  Stride 1 only.
#include "mie_conv.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int FC_CH = 8;     // staged channels per pixel
constexpr int FC_PS = 9;     // LDS floats per staged pixel (odd: the 32 pixels of a block fall on distinct banks)

template <typename T, int K, int S, bool UP = false>
__global__ __launch_bounds__(256) void k_conv_fewcin(ConvArgsT<T> a) {
  static_assert(!UP || S == 1, "the up-sampling form is stride 1");
  constexpr int IT = 7 * S + K;                  // input tile edge incl. halo
  constexpr int NPIX = IT * IT;
  constexpr int IN_F = NPIX * FC_PS;
  constexpr int W_F = K * K * FC_CH * 32;
  constexpr int RED_F = 2 * 64 * 32;             // the accumulators of the two tap halves, parked for the epilogue
  constexpr int SMEM_F = (IN_F + W_F > RED_F) ? IN_F + W_F : RED_F;      // (they reuse the staging area)
  __shared__ float smem[SMEM_F];
  float* const s_in = smem;
  float* const s_w = smem + IN_F;

  int n, y0, x0;
  const int tk = mie_pick_tile(a.ts, blockIdx.x + conv_args_entry_zero(a), n, y0, x0);
  if (tk == 0) return;
  const int tid = threadIdx.x;
  const int hout = a.ts.h, wout = a.ts.w, cout = a.cout, cin = a.c1;
  const int co0 = blockIdx.y * 32;
  if (tk == 2) {   // stale tile: zero this workgroup's channel slab
    for (int idx = tid; idx < 64 * 8; idx += 256) {        // groups of four channels
      const int p = idx >> 3, col = 4 * (idx & 7);
      const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
      if (oy < hout && ox < wout)
        mie_st4(a.out, (((long long)n * hout + oy) * wout + ox) * cout + co0 + col, make_float4(0.f, 0.f, 0.f, 0.f));
    }
    return;
  }

  // pixels of this thread's two epilogue groups that lie in the output pixel mask (elsewhere the sums are exactly
  // zero: no reservoir access, a zero delta); the bytes are asked for before the staging loads
  bool live[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int p = (tid + 256 * i) >> 3;
    const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
    live[i] = oy < hout && ox < wout && (a.refresh || a.ts.pixmask[((long long)n * hout + oy) * wout + ox] != 0);
  }

  // ---- stage the input tile (fp32, 8 channels per pixel) and the filter slab ---------------------
  // Every global load of the thread is issued before the first LDS store (compile-time trip counts, fully
  // unrolled): one memory round trip for the whole staging instead of one per loop iteration.
  const int iy0 = y0 * S - a.pad, ix0 = x0 * S - a.pad;
  constexpr int NIN = (NPIX * FC_CH + 255) / 256;
  float vin[NIN], vw[K * K];
  {
    const int col = tid & 31, ch = (tid >> 5) & 7;           // filter: thread = (channel, column), one load per tap
    const float* wp = a.filt + (long long)ch * (K * K) * cout + co0 + col;
#pragma unroll
    for (int tap = 0; tap < K * K; ++tap) vw[tap] = (ch < cin) ? wp[(long long)tap * cout] : 0.f;
  }
#pragma unroll
  for (int i = 0; i < NIN; ++i) {
    const int idx = tid + 256 * i;
    const int pix = idx >> 3, ch = idx & 7;
    const int iy = iy0 + pix / IT, ix = ix0 + pix % IT;
    float v = 0.f;
    if (pix < NPIX && ch < cin && iy >= 0 && iy < a.h_in && ix >= 0 && ix < a.w_in) {
      if constexpr (UP) {
        const int h_lo = a.h_in >> 1, w_lo = a.w_in >> 1;
        int r[2], q[2];
        float lr[2], lq[2];
        conv_up2x_coef(iy, h_lo, r[0], r[1], lr[0], lr[1]);
        conv_up2x_coef(ix, w_lo, q[0], q[1], lq[0], lq[1]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const long long po = ((long long)n * h_lo + r[j >> 1]) * w_lo + q[j & 1];
          if (a.xm == nullptr || a.xm[po]) v += lr[j >> 1] * lq[j & 1] * mie_ld(a.x, po * cin + ch);
        }
      } else {
        const long long po = ((long long)n * a.h_in + iy) * a.w_in + ix;
        if (a.xm == nullptr || a.xm[po]) v = mie_ld(a.x, po * cin + ch);
      }
    }
    vin[i] = v;
  }
#pragma unroll
  for (int tap = 0; tap < K * K; ++tap) s_w[tap * 256 + tid] = vw[tap];
#pragma unroll
  for (int i = 0; i < NIN; ++i) {
    const int idx = tid + 256 * i;
    if ((idx >> 3) < NPIX) s_in[(idx >> 3) * FC_PS + (idx & 7)] = vin[i];
  }
  __syncthreads();

  // ---- contraction ---------------------------------------------------------------------------------
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int mb = wave & 1, th = wave >> 1;
  const int prow = mb * 4 + (l32 >> 3), pcol = l32 & 7;
  const float* pa = s_in + ((prow * S) * IT + pcol * S) * FC_PS + half;
  const float* pb = s_w + half * 32 + l32;
  const int npair = (cin + 1) >> 1;
  v16f acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  for (int tap = th; tap < K * K; tap += 2) {
    const int dy = tap / K, dx = tap - dy * K;
    const float* ta = pa + (dy * IT + dx) * FC_PS;
    const float* tb = pb + tap * (FC_CH * 32);
    for (int p = 0; p < npair; ++p)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ta[2 * p], tb[2 * p * 32], acc, 0, 0, 0);
  }
  __syncthreads();                       // every wave is done with the staged operands
  // ---- epilogue: the two tap halves park their accumulators in LDS; a thread then owns groups of four adjacent
  // output channels of a pixel (16-byte reads of the two partial sums, 16-byte reservoir accesses, 16- / 8-byte
  // delta accesses; all reservoir / addend loads of the thread as one batch, then the stores)
  float* red = smem + th * (64 * 32);
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int p = mb * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
    red[p * 32 + l32] = acc[r];
  }
  __syncthreads();
  long long off[2];
  int co[2];
  bool ok[2];
  float4 v[2], r0[2], add[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int idx = tid + 256 * i;
    const int p = idx >> 3, col = 4 * (idx & 7);
    const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
    ok[i] = oy < hout && ox < wout;
    off[i] = (((long long)n * hout + oy) * wout + ox) * cout + co0 + col;
    co[i] = co0 + col;
    const float4 s0 = *reinterpret_cast<const float4*>(&smem[4 * idx]);
    const float4 s1 = *reinterpret_cast<const float4*>(&smem[64 * 32 + 4 * idx]);
    v[i] = make_float4(s0.x + s1.x, s0.y + s1.y, s0.z + s1.z, s0.w + s1.w);
  }
  conv_epilogue_load4<T, 2>(a, off, live, r0, add);
  conv_epilogue_store4<T, 2>(a, off, co, ok, v, r0, add, live);
}

template <typename T>
bool launch_fewcin(const ConvArgsT<T>& a, int k, int s, unsigned cap, hipStream_t st) {
  if (a.x2 != nullptr || a.c1 < 1 || a.c1 > FC_CH || a.cout % 32 != 0) return false;
  const dim3 grid(cap, a.cout / 32), block(256);
  switch (k * 10 + s) {
    case 31: hipLaunchKernelGGL((k_conv_fewcin<T, 3, 1>), grid, block, 0, st, a); return true;
    case 32: hipLaunchKernelGGL((k_conv_fewcin<T, 3, 2>), grid, block, 0, st, a); return true;
    case 51: hipLaunchKernelGGL((k_conv_fewcin<T, 5, 1>), grid, block, 0, st, a); return true;
    case 52: hipLaunchKernelGGL((k_conv_fewcin<T, 5, 2>), grid, block, 0, st, a); return true;
    default: return false;
  }
}

template <typename T>
bool launch_fewcin_up(const ConvArgsT<T>& a, int k, unsigned cap, hipStream_t st) {
  if (a.x2 != nullptr || a.c1 < 1 || a.c1 > FC_CH || a.cout % 32 != 0 || a.pad != k / 2) return false;
  const dim3 grid(cap, a.cout / 32), block(256);
  switch (k) {
    case 3: hipLaunchKernelGGL((k_conv_fewcin<T, 3, 1, true>), grid, block, 0, st, a); return true;
    case 5: hipLaunchKernelGGL((k_conv_fewcin<T, 5, 1, true>), grid, block, 0, st, a); return true;
    default: return false;
  }
}

}  // namespace

bool mie_launch_conv_fewcin_up(const ConvArgsT<float>& a, int k, unsigned cap, hipStream_t st) {
  return launch_fewcin_up(a, k, cap, st);
}
bool mie_launch_conv_fewcin_up(const ConvArgsT<mie_bf16>& a, int k, unsigned cap, hipStream_t st) {
  return launch_fewcin_up(a, k, cap, st);
}
bool mie_launch_conv_fewcin(const ConvArgsT<float>& a, int k, int s, unsigned cap, hipStream_t st) {
  return launch_fewcin(a, k, s, cap, st);
}
bool mie_launch_conv_fewcin(const ConvArgsT<mie_bf16>& a, int k, int s, unsigned cap, hipStream_t st) {
  return launch_fewcin(a, k, s, cap, st);
}
