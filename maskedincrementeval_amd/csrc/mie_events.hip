// Event front end: raw events -> voxel-grid (or polarity-histogram) frames and frame DELTAS in the
// layout the incremental network consumes (fp32 NHWC + uint8 pixel mask), without forming two dense
// frames and subtracting them.
//
// One thread per event.  An event (t, x, y, p) lies in a window (start, start + delta_t) or not;
// inside, it adds p*(1-dt) to bin floor(ts) and p*dt to the next bin, ts = (bins-1)*(t-start)/delta_t
// (data_fetchers/utils/util.py:90-107 of the reference).  The delta between two windows is the sum
// over events of (contribution to the new window) - (contribution to the old one): every event of
// either window is visited once and issues at most 4 atomic adds per target pixel.  Reflection
// padding (run_e2depth_continuous_dataset.py:49) is linear, so it is applied to the scatter targets:
// an event near the border also lands on its mirror pixels.
//
// The kernels are bandwidth-trivial (a window holds 1e4..1e6 events, 32 bytes each); what matters is
// that the dense subtraction of two frames and the later any-over-channels mask pass disappear.
// Floating-point atomics make the summation order, and with it the last bits of a pixel that
// receives several events, vary from run to run; the histogram kind adds integers and is exact.
#include "mie_common.h"

namespace {

struct EventArgs {
  const double* ev;        // [n_events][4] = (t, x, y, p)
  int n_events;
  int kind, bins, h, w;    // sensor size
  int pl, pr, pt, pb;      // reflection padding
  double t_scale, start_old, start_new, delta_t;
  int delta;               // 1: new - old, 0: new only
  float* out;              // [h + pt + pb][w + pl + pr][channels]
  uint8_t* pixmask;        // [h + pt + pb][w + pl + pr]
};

// Padded coordinates an input coordinate lands on: itself, plus its mirror images in the left/top and
// right/bottom border (reflection without repeating the edge sample).  Returns how many.
__device__ __forceinline__ int reflect_targets(int v, int size, int lo, int hi, int (&dst)[3]) {
  int n = 0;
  dst[n++] = v + lo;
  if (v >= 1 && v <= lo) dst[n++] = lo - v;
  if (v <= size - 2 && v >= size - 1 - hi) dst[n++] = lo + size + (size - 2 - v);
  return n;
}

__global__ __launch_bounds__(256) void k_events_clear(float* __restrict__ out, long long n,
                                                      uint8_t* __restrict__ mask, long long m) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long stride = (long long)gridDim.x * 256;
  float4* out4 = reinterpret_cast<float4*>(out);
  uint32_t* mask4 = reinterpret_cast<uint32_t*>(mask);
  for (long long j = i; j < n / 4; j += stride) out4[j] = make_float4(0.f, 0.f, 0.f, 0.f);
  for (long long j = i; j < m / 4; j += stride) mask4[j] = 0u;
  if (i < (n & 3)) out[(n & ~3LL) + i] = 0.f;         // tails
  if (i < (m & 3)) mask[(m & ~3LL) + i] = 0;
}

__global__ __launch_bounds__(256) void k_events_scatter(EventArgs a) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= a.n_events) return;
  const double t = a.ev[4LL * i] * a.t_scale;
  const double xd = a.ev[4LL * i + 1], yd = a.ev[4LL * i + 2];
  double p = a.ev[4LL * i + 3];
  if (!(xd >= 0.0 && xd < (double)a.w && yd >= 0.0 && yd < (double)a.h)) return;   // off the sensor (or NaN)
  const int x = (int)xd, y = (int)yd;
  const int channels = a.kind == MIE_EVENTS_HISTOGRAM ? 2 : a.bins;
  const int wp = a.w + a.pl + a.pr;

  int ch[4];
  float val[4];
  int nc = 0;
  for (int pass = 0; pass < 2; ++pass) {
    if (pass == 1 && !a.delta) break;
    const double start = pass == 0 ? a.start_new : a.start_old;
    const float sign = pass == 0 ? 1.f : -1.f;
    if (!(t > start && t < start + a.delta_t)) continue;
    if (a.kind == MIE_EVENTS_HISTOGRAM) {
      // event_histogram (util.py:62-75): channel 0 counts p == -1, channel 1 counts p == +1
      if (p == 1.0 || p == -1.0) { ch[nc] = p == 1.0 ? 1 : 0; val[nc++] = sign; }
    } else {
      const double pol = p == 0.0 ? -1.0 : p;                       // util.py:94
      const double ts = (double)(a.bins - 1) * (t - start) / a.delta_t;
      const int ti = (int)ts;
      const double dt = ts - (double)ti;
      if (ti < a.bins) { ch[nc] = ti; val[nc++] = sign * (float)(pol * (1.0 - dt)); }
      if (ti + 1 < a.bins) { ch[nc] = ti + 1; val[nc++] = sign * (float)(pol * dt); }
    }
  }
  if (nc == 0) return;
  int xs[3], ys[3];
  const int nx = reflect_targets(x, a.w, a.pl, a.pr, xs);
  const int ny = reflect_targets(y, a.h, a.pt, a.pb, ys);
  for (int iy = 0; iy < ny; ++iy)
    for (int ix = 0; ix < nx; ++ix) {
      const long long pix = (long long)ys[iy] * wp + xs[ix];
      a.pixmask[pix] = 1;
      for (int c = 0; c < nc; ++c) atomicAdd(a.out + pix * channels + ch[c], val[c]);
    }
}

// fp32 sums -> bf16 elements (round to nearest even), four per thread; the sums are zero where no event landed
__global__ __launch_bounds__(256) void k_events_round(const float* __restrict__ acc, long long n, mie_bf16* __restrict__ out) {
  const long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i + 4 <= n) {
    const float4 v = *reinterpret_cast<const float4*>(acc + i);
    mie_st4(out, i, v);
  } else {
    for (long long j = i; j < n; ++j) out[j] = (mie_bf16)acc[j];
  }
}

}  // namespace

extern "C" int mie_events_to_frame(const double* events, int n_events, int kind, int num_bins,
                                   int height, int width, int pad_left, int pad_right, int pad_top,
                                   int pad_bottom, double t_scale, double start_old,
                                   double start_new, double delta_t, int delta, float* out,
                                   uint8_t* pixmask, void* stream) {
  mie_clear_error();
  const char* who = "mie_events_to_frame";
  MIE_REQUIRE(out && pixmask, MIE_ERR_INVALID_ARG, "%s: NULL output", who);
  MIE_REQUIRE(n_events >= 0 && (events || n_events == 0), MIE_ERR_INVALID_ARG,
              "%s: %d events at a NULL pointer", who, n_events);
  MIE_REQUIRE(kind == MIE_EVENTS_VOXEL || kind == MIE_EVENTS_HISTOGRAM, MIE_ERR_UNSUPPORTED,
              "%s: unknown frame kind %d", who, kind);
  MIE_REQUIRE(height > 0 && width > 0 && (kind == MIE_EVENTS_HISTOGRAM || (num_bins > 0 && num_bins <= 64)),
              MIE_ERR_INVALID_ARG, "%s: bad geometry (bins %d, %dx%d)", who, num_bins, height, width);
  MIE_REQUIRE(pad_left >= 0 && pad_right >= 0 && pad_top >= 0 && pad_bottom >= 0 &&
                  pad_left < width && pad_right < width && pad_top < height && pad_bottom < height,
              MIE_ERR_INVALID_ARG, "%s: reflection padding must be smaller than the frame", who);
  MIE_REQUIRE(delta_t > 0.0 && t_scale > 0.0, MIE_ERR_INVALID_ARG,
              "%s: window length and time scale must be positive", who);
  const int channels = kind == MIE_EVENTS_HISTOGRAM ? 2 : num_bins;
  const long long pixels = (long long)(height + pad_top + pad_bottom) * (width + pad_left + pad_right);
  MIE_REQUIRE(pixels * channels < (1LL << 31), MIE_ERR_CAPACITY, "%s: frame too large", who);
  MIE_REQUIRE(mie_aligned(events, 8), MIE_ERR_INVALID_ARG, "%s: events must be 8-byte aligned", who);
  MIE_REQUIRE(mie_aligned(out, 16) && mie_aligned(pixmask, 4), MIE_ERR_INVALID_ARG,
              "%s: out must be 16-byte and pixmask 4-byte aligned", who);
  hipStream_t s = (hipStream_t)stream;
  const long long n4 = pixels * channels / 4 + 1;
  const unsigned clear_blocks = (unsigned)((n4 + 255) / 256 < 2048 ? (n4 + 255) / 256 : 2048);
  hipLaunchKernelGGL(k_events_clear, dim3(clear_blocks), dim3(256), 0, s, out, pixels * channels, pixmask,
                     pixels);
  int rc = mie_check_launch(who);
  if (rc != MIE_OK || n_events == 0) return rc;
  EventArgs a;
  a.ev = events; a.n_events = n_events; a.kind = kind; a.bins = num_bins; a.h = height; a.w = width;
  a.pl = pad_left; a.pr = pad_right; a.pt = pad_top; a.pb = pad_bottom;
  a.t_scale = t_scale; a.start_old = start_old; a.start_new = start_new; a.delta_t = delta_t;
  a.delta = delta ? 1 : 0; a.out = out; a.pixmask = pixmask;
  hipLaunchKernelGGL(k_events_scatter, dim3((unsigned)((n_events + 255) / 256)), dim3(256), 0, s, a);
  return mie_check_launch(who);
}

extern "C" int mie_events_to_frame_bf16(const double* events, int n_events, int kind, int num_bins,
                                        int height, int width, int pad_left, int pad_right, int pad_top,
                                        int pad_bottom, double t_scale, double start_old,
                                        double start_new, double delta_t, int delta, float* sums,
                                        void* out, uint8_t* pixmask, void* stream) {
  const char* who = "mie_events_to_frame_bf16";
  int rc = mie_events_to_frame(events, n_events, kind, num_bins, height, width, pad_left, pad_right, pad_top,
                               pad_bottom, t_scale, start_old, start_new, delta_t, delta, sums, pixmask, stream);
  if (rc != MIE_OK) return rc;
  MIE_REQUIRE(out != nullptr && mie_aligned(out, 8), MIE_ERR_INVALID_ARG, "%s: out must be 8-byte aligned", who);
  MIE_REQUIRE(out != (void*)sums, MIE_ERR_INVALID_ARG, "%s: out and sums are different buffers", who);
  const int channels = kind == MIE_EVENTS_HISTOGRAM ? 2 : num_bins;
  const long long n = (long long)(height + pad_top + pad_bottom) * (width + pad_left + pad_right) * channels;
  hipLaunchKernelGGL(k_events_round, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, (hipStream_t)stream, sums, n,
                     reinterpret_cast<mie_bf16*>(out));
  return mie_check_launch(who);
}
