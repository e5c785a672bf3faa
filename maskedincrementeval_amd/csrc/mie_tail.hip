// The ops behind a classifier tail on deltas: per-channel scale (the linear part of an eval-mode batch
// norm), adaptive average pooling and the fully connected layer.  All three are linear, so they apply
// to the delta directly; what the masks buy is that inactive pixels / zero features are not read.
//
//   scale   : out = d * scale[c] over the active tiles of the set (clean zeros elsewhere in them)
//   avgpool : out[n, oy, ox, c] = mean of d over torch's adaptive window; inactive pixels add nothing
//   linear  : out[n, o] = sum_i d[n, i] * W[o, i]; features with d == 0 skip their row of W^T
//
// All are bandwidth-bound and tiny at the sizes classifier tails have (7x7x512 planes, 512x1000
// weights): what matters is that they are one launch each and leave no dense pass behind.
#include "mie_common.h"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void k_scale_incr(TileSetDev ts, const T* __restrict__ din,
                                                    const float* __restrict__ scale,
                                                    T* __restrict__ dout, int c) {
  int n, y0, x0;
  const int tk = mie_pick_tile(ts, blockIdx.x, n, y0, x0);
  if (tk == 0) return;
  const int total = 64 * c;
  for (int idx = threadIdx.x; idx < total; idx += 256) {
    const int px = idx / c, ch = idx - px * c;
    const int y = y0 + (px >> 3), x = x0 + (px & 7);
    if (y >= ts.h || x >= ts.w) continue;
    const long long pix = ((long long)n * ts.h + y) * ts.w + x;
    float v = 0.f;
    if (tk == 1 && ts.pixmask[pix]) v = mie_ld(din, pix * c + ch) * scale[ch];
    mie_st(dout, pix * c + ch, v);
  }
}

// torch's adaptive pooling window of output index o: [floor(o*in/out), ceil((o+1)*in/out))
__device__ __forceinline__ void adaptive_window(int o, int in, int out, int& lo, int& hi) {
  lo = (int)(((long long)o * in) / out);
  hi = (int)(((long long)(o + 1) * in + out - 1) / out);
}

template <typename T>
__global__ __launch_bounds__(256) void k_avgpool_incr(const T* __restrict__ din,
                                                      const uint8_t* __restrict__ mask, int h, int w,
                                                      int c, int oh, int ow, T* __restrict__ dout) {
  const int n = blockIdx.y, o = blockIdx.x;
  const int oy = o / ow, ox = o - oy * ow;
  int ylo, yhi, xlo, xhi;
  adaptive_window(oy, h, oh, ylo, yhi);
  adaptive_window(ox, w, ow, xlo, xhi);
  const float inv = 1.f / (float)((yhi - ylo) * (xhi - xlo));
  for (int ch = threadIdx.x; ch < c; ch += 256) {
    float acc = 0.f;
    for (int y = ylo; y < yhi; ++y)
      for (int x = xlo; x < xhi; ++x) {
        const long long pix = ((long long)n * h + y) * w + x;
        if (mask == nullptr || mask[pix]) acc += mie_ld(din, pix * c + ch);   // uniform branch
      }
    mie_st(dout, (((long long)n * oh + oy) * ow + ox) * c + ch, acc * inv);
  }
}

// One workgroup = 64 output features of one sample; its 4 waves split the input features 4 ways in
// blocks of 64.  A wave loads 64 deltas (one per lane), and for every non-zero one -- found with a
// ballot, so the loop is uniform -- adds delta * W^T[i][o..o+63], a coalesced 256-byte row segment.
// The four partial sums meet in LDS and are added in wave order (bit-reproducible).
template <typename T>
__global__ __launch_bounds__(256) void k_linear_incr(const T* __restrict__ din,
                                                     const float* __restrict__ wt, int f_in,
                                                     int f_out, T* __restrict__ dout) {
  __shared__ float part[4][64];
  const int n = blockIdx.y;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int o = blockIdx.x * 64 + lane;
  const bool o_ok = o < f_out;
  const T* drow = din + (long long)n * f_in;
  float acc = 0.f;
  for (int i0 = wave * 64; i0 < f_in; i0 += 256) {
    const int i = i0 + lane;
    const float d = (i < f_in) ? mie_ld(drow, i) : 0.f;
    unsigned long long live = __ballot(d != 0.f);
    while (live) {
      const int j = __builtin_amdgcn_readfirstlane(__builtin_ctzll(live));
      live &= live - 1;
      const float dj = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, d), j));
      if (o_ok) acc += dj * wt[(long long)(i0 + j) * f_out + o];
    }
  }
  part[wave][lane] = acc;
  __syncthreads();
  if (wave == 0 && o_ok)
    mie_st(dout, (long long)n * f_out + o, ((part[0][lane] + part[1][lane]) + part[2][lane]) + part[3][lane]);
}

#define MIE_TAIL_DTYPE_OK(dtype, who)                                                                 \
  MIE_REQUIRE((dtype) == MIE_DTYPE_F32 || (dtype) == MIE_DTYPE_BF16, MIE_ERR_UNSUPPORTED,              \
              "%s: unknown delta dtype %d", who, (int)(dtype))

}  // namespace

extern "C" int mie_scale_incr(const void* in_delta, const float* scale, void* out_delta, int c,
                              const mie_tileset* ts, int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_scale_incr";
  int rc = mie_check_tileset(ts, who);
  if (rc != MIE_OK) return rc;
  MIE_TAIL_DTYPE_OK(dtype, who);
  MIE_REQUIRE(c > 0 && c <= 65536, MIE_ERR_INVALID_ARG, "%s: channel count %d out of range", who, c);
  MIE_REQUIRE(in_delta && scale && out_delta, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(mie_aligned(in_delta, 4) && mie_aligned(out_delta, 4) && mie_aligned(scale, 4),
              MIE_ERR_INVALID_ARG, "%s: buffers must be 4-byte aligned", who);
  const TileSetDev d = mie_dev_tileset(ts);
  const unsigned grid = (unsigned)mie_tile_capacity(ts->n, ts->h, ts->w);
  if (dtype == MIE_DTYPE_BF16)
    hipLaunchKernelGGL(k_scale_incr<mie_bf16>, dim3(grid), dim3(256), 0, (hipStream_t)stream, d,
                       (const mie_bf16*)in_delta, scale, (mie_bf16*)out_delta, c);
  else
    hipLaunchKernelGGL(k_scale_incr<float>, dim3(grid), dim3(256), 0, (hipStream_t)stream, d,
                       (const float*)in_delta, scale, (float*)out_delta, c);
  return mie_check_launch(who);
}

extern "C" int mie_avgpool_incr(const void* in_delta, const uint8_t* in_mask, int n, int h_in,
                                int w_in, int c, int h_out, int w_out, void* out_delta, int dtype,
                                void* stream) {
  mie_clear_error();
  const char* who = "mie_avgpool_incr";
  MIE_TAIL_DTYPE_OK(dtype, who);
  MIE_REQUIRE(in_delta && out_delta, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(n > 0 && n <= 65535 && h_in > 0 && w_in > 0 && c > 0 && h_out > 0 && w_out > 0,
              MIE_ERR_INVALID_ARG, "%s: bad geometry (n=%d in %dx%d out %dx%d c=%d)", who, n, h_in, w_in,
              h_out, w_out, c);
  MIE_REQUIRE((long long)n * h_in * w_in * c < (1LL << 40) && (long long)h_out * w_out < (1LL << 30),
              MIE_ERR_CAPACITY, "%s: too large", who);
  MIE_REQUIRE(mie_aligned(in_delta, 4) && mie_aligned(out_delta, 4), MIE_ERR_INVALID_ARG,
              "%s: buffers must be 4-byte aligned", who);
  const dim3 grid((unsigned)(h_out * w_out), (unsigned)n);
  if (dtype == MIE_DTYPE_BF16)
    hipLaunchKernelGGL(k_avgpool_incr<mie_bf16>, grid, dim3(256), 0, (hipStream_t)stream,
                       (const mie_bf16*)in_delta, in_mask, h_in, w_in, c, h_out, w_out, (mie_bf16*)out_delta);
  else
    hipLaunchKernelGGL(k_avgpool_incr<float>, grid, dim3(256), 0, (hipStream_t)stream,
                       (const float*)in_delta, in_mask, h_in, w_in, c, h_out, w_out, (float*)out_delta);
  return mie_check_launch(who);
}

extern "C" int mie_linear_incr(const void* in_delta, int n, int f_in, const float* weight_t,
                               int f_out, void* out_delta, int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_linear_incr";
  MIE_TAIL_DTYPE_OK(dtype, who);
  MIE_REQUIRE(in_delta && weight_t && out_delta, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(n > 0 && n <= 65535 && f_in > 0 && f_out > 0, MIE_ERR_INVALID_ARG,
              "%s: sizes out of range (n=%d f_in=%d f_out=%d)", who, n, f_in, f_out);
  MIE_REQUIRE((long long)f_in * f_out < (1LL << 40), MIE_ERR_CAPACITY, "%s: weight too large", who);
  MIE_REQUIRE(mie_aligned(in_delta, 4) && mie_aligned(out_delta, 4) && mie_aligned(weight_t, 4),
              MIE_ERR_INVALID_ARG, "%s: buffers must be 4-byte aligned", who);
  MIE_REQUIRE(in_delta != out_delta, MIE_ERR_INVALID_ARG, "%s: out_delta must not alias in_delta", who);
  const dim3 grid((unsigned)mie_div_up(f_out, 64), (unsigned)n);
  if (dtype == MIE_DTYPE_BF16)
    hipLaunchKernelGGL(k_linear_incr<mie_bf16>, grid, dim3(256), 0, (hipStream_t)stream,
                       (const mie_bf16*)in_delta, weight_t, f_in, f_out, (mie_bf16*)out_delta);
  else
    hipLaunchKernelGGL(k_linear_incr<float>, grid, dim3(256), 0, (hipStream_t)stream,
                       (const float*)in_delta, weight_t, f_in, f_out, (float*)out_delta);
  return mie_check_launch(who);
}
