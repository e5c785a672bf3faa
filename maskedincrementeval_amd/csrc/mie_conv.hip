// Masked convolution of a delta over active 8x8 output tiles (gfx950).
//
// Code paths, one per arithmetic regime:
//   mfma    : input channels in whole staging chunks (32 fp32 / 64 bf16 channels; 16 / 32 for 7x7
//             and as the fallback depth at stride 2) and Cout % 32 == 0 -- per-tile implicit GEMM
//             on the matrix cores (mie_conv_mfma_impl.h), optionally with the ConvLSTM gate chain
//             as its epilogue.
//   valu    : any shape -- thread = one output channel x 16 pixels, input tile
//             staged in LDS and read as wave-wide broadcasts.
//   smallco : Cout <= 4 (prediction / flow heads) -- thread = one pixel; 1x1 convs of that kind
//             walk whole NHWC rows with 4 lanes per pixel.
//   tconv   : transposed conv, gather form.
// All paths share the epilogue: plain delta store, the fused reservoir update + activation
// increment, or (dense refresh) bias + activation + reservoir fill.
#include "mie_common.h"
#include "mie_conv.h"
#include <mutex>

namespace {

// ---------------------------------------------------------------------------------
// VALU path.  Block = 256 threads = 64 output channels x 4 pixel groups (two
// tile rows each).  CC input channels per LDS stage.
// ---------------------------------------------------------------------------------
template <typename T, int K, int S>
__global__ __launch_bounds__(256) void k_conv_valu(ConvArgsT<T> a) {
  constexpr int IT = 7 * S + K;  // input tile edge incl. halo
  constexpr int CC = 8;
  __shared__ float s_in[IT * IT * CC];
  int n, y0, x0;
  const int tk = mie_pick_tile(a.ts, blockIdx.x, n, y0, x0);
  if (tk == 0) return;
  const int co = blockIdx.y * 64 + (threadIdx.x & 63);
  const int pg = threadIdx.x >> 6;
  const int hout = a.ts.h, wout = a.ts.w;
  if (tk == 2) {
    if (co < a.cout)
      for (int p = 0; p < 16; ++p) {
        const int oy = y0 + 2 * pg + (p >> 3), ox = x0 + (p & 7);
        if (oy < hout && ox < wout) mie_st(a.out, (((long long)n * hout + oy) * wout + ox) * a.cout + co, 0.f);
      }
    return;
  }
  float acc[16];
#pragma unroll
  for (int p = 0; p < 16; ++p) acc[p] = 0.f;
  const int iy0 = y0 * S - a.pad, ix0 = x0 * S - a.pad;

  for (int src = 0; src < 2; ++src) {
    const T* xin = src ? a.x2 : a.x;
    const uint8_t* xm = src ? a.x2m : a.xm;
    const int cs = src ? a.c2 : a.c1;
    const int fbase = src ? a.c1 : 0;
    if (xin == nullptr || cs == 0) continue;
    for (int ci0 = 0; ci0 < cs; ci0 += CC) {
      __syncthreads();
      for (int idx = threadIdx.x; idx < IT * IT * CC; idx += 256) {
        const int pix = idx / CC, cc = idx % CC;
        const int iy = iy0 + pix / IT, ix = ix0 + pix % IT;
        float v = 0.f;
        if (ci0 + cc < cs && iy >= 0 && iy < a.h_in && ix >= 0 && ix < a.w_in) {
          const long long po = ((long long)n * a.h_in + iy) * a.w_in + ix;
          if (xm == nullptr || xm[po]) v = mie_ld(xin, po * cs + ci0 + cc);
        }
        s_in[idx] = v;
      }
      __syncthreads();
      const int nci = (cs - ci0 < CC) ? cs - ci0 : CC;
      for (int cc = 0; cc < nci; ++cc) {
        // all K*K filter taps of this input channel first (independent loads, one latency), then the
        // multiply-adds: a load inside the tap loop would expose the L2 latency K*K times
        const float* wp = a.filt + (long long)(fbase + ci0 + cc) * K * K * a.cout + co;
        float wv[K * K];
#pragma unroll
        for (int t = 0; t < K * K; ++t) wv[t] = (co < a.cout) ? wp[t * a.cout] : 0.f;
#pragma unroll
        for (int ky = 0; ky < K; ++ky)
#pragma unroll
          for (int kx = 0; kx < K; ++kx) {
#pragma unroll
            for (int p = 0; p < 16; ++p) {
              const int py = 2 * pg + (p >> 3), px = p & 7;
              acc[p] += s_in[((py * S + ky) * IT + px * S + kx) * CC + cc] * wv[ky * K + kx];
            }
          }
      }
    }
  }
  if (co < a.cout) {
#pragma unroll
    for (int p = 0; p < 16; ++p) {
      const int oy = y0 + 2 * pg + (p >> 3), ox = x0 + (p & 7);
      if (oy < hout && ox < wout)
        conv_store(a, (((long long)n * hout + oy) * wout + ox) * a.cout + co, co, acc[p]);
    }
  }
}

// ---------------------------------------------------------------------------------
// Small-Cout path (Cout <= 4): one wave per tile, lane = output pixel.
// ---------------------------------------------------------------------------------
template <typename T, int K, int S>
__global__ __launch_bounds__(64) void k_conv_smallco(ConvArgsT<T> a) {
  int n, y0, x0;
  const int tk = mie_pick_tile(a.ts, blockIdx.x, n, y0, x0);
  if (tk == 0) return;
  const int lane = threadIdx.x;
  const int oy = y0 + (lane >> 3), ox = x0 + (lane & 7);
  const int hout = a.ts.h, wout = a.ts.w;
  if (oy >= hout || ox >= wout) return;
  const long long obase = (((long long)n * hout + oy) * wout + ox) * a.cout;
  if (tk == 2) {
    for (int co = 0; co < a.cout; ++co) mie_st(a.out, obase + co, 0.f);
    return;
  }
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int src = 0; src < 2; ++src) {
    const T* xin = src ? a.x2 : a.x;
    const uint8_t* xm = src ? a.x2m : a.xm;
    const int cs = src ? a.c2 : a.c1;
    const int fbase = src ? a.c1 : 0;
    if (xin == nullptr || cs == 0) continue;
    for (int ky = 0; ky < K; ++ky) {
      const int iy = oy * S - a.pad + ky;
      if (iy < 0 || iy >= a.h_in) continue;
      for (int kx = 0; kx < K; ++kx) {
        const int ix = ox * S - a.pad + kx;
        if (ix < 0 || ix >= a.w_in) continue;
        const long long po = ((long long)n * a.h_in + iy) * a.w_in + ix;
        if (xm != nullptr && !xm[po]) continue;
        const T* xr = xin + po * cs;
        for (int ci = 0; ci < cs; ++ci) {
          const float xv = mie_ld(xr, ci);
          const float* wp = a.filt + ((long long)(fbase + ci) * K * K + ky * K + kx) * a.cout;
          for (int co = 0; co < a.cout; ++co) acc[co] += xv * wp[co];
        }
      }
    }
  }
  for (int co = 0; co < a.cout; ++co) conv_store(a, obase + co, co, acc[co]);
}

// ---------------------------------------------------------------------------------
// 1x1 stride-1 conv with Cout <= 4 and Cin % 4 == 0 (prediction layer 32 -> 1, flow heads): pure
// bandwidth work.  4 lanes share one pixel and walk its NHWC row in 16-byte (fp32) / 8-byte
// (bf16) pieces, so a wave reads whole 8-pixel tile rows as contiguous segments; the partial
// sums meet through two lane exchanges.  Lane `sub` of a pixel stores output channel `sub`.
// ---------------------------------------------------------------------------------
static __device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
static __device__ __forceinline__ float4 load4(const mie_bf16* p) {
  const mie_bf16x4 b = *reinterpret_cast<const mie_bf16x4*>(p);
  return make_float4((float)b[0], (float)b[1], (float)b[2], (float)b[3]);
}

template <typename T>
__global__ __launch_bounds__(256) void k_conv1x1_smallco(ConvArgsT<T> a) {
  int n, y0, x0;
  const int tk = mie_pick_tile(a.ts, blockIdx.x + conv_args_entry_zero(a), n, y0, x0);
  if (tk == 0) return;
  const int px = threadIdx.x >> 2, sub = threadIdx.x & 3;
  const int oy = y0 + (px >> 3), ox = x0 + (px & 7);
  const int hout = a.ts.h, wout = a.ts.w;
  const bool inb = oy < hout && ox < wout;
  const long long po = ((long long)n * hout + oy) * wout + ox;      // input pixel = output pixel
  if (tk == 2) {
    if (inb && sub < a.cout) mie_st(a.out, po * a.cout + sub, 0.f);
    return;
  }
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int src = 0; src < 2; ++src) {        // x feeds filter rows [0, c1), x2 rows [c1, c1 + c2)
    const T* xin = src ? a.x2 : a.x;
    const uint8_t* xm = src ? a.x2m : a.xm;
    const int cs = src ? a.c2 : a.c1;
    if (xin == nullptr || !inb || (xm != nullptr && !xm[po])) continue;
    const T* xr = xin + po * cs;
    const float* wrow = a.filt + (long long)(src ? a.c1 : 0) * a.cout;
    for (int v = sub; v < (cs >> 2); v += 4) {
      const float4 x = load4(xr + 4 * v);
      const float* wp = wrow + (long long)(4 * v) * a.cout;
      for (int co = 0; co < a.cout; ++co)
        acc[co] += x.x * wp[co] + x.y * wp[a.cout + co] + x.z * wp[2 * a.cout + co] + x.w * wp[3 * a.cout + co];
    }
  }
#pragma unroll
  for (int co = 0; co < 4; ++co) {           // every lane of the wave takes part
    acc[co] += __shfl_xor(acc[co], 1);
    acc[co] += __shfl_xor(acc[co], 2);
  }
  const float mine = sub == 0 ? acc[0] : (sub == 1 ? acc[1] : (sub == 2 ? acc[2] : acc[3]));
  if (inb && sub < a.cout) conv_store(a, po * a.cout + sub, sub, mine);
}

// ---------------------------------------------------------------------------------
// Transposed conv, gather form.  Thread = one output channel x 16 pixels;
// input values are wave-uniform loads (every lane of a wave reads the same
// address), filter rows are coalesced over the output channel.
// ---------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void k_tconv_valu(ConvArgsT<T> a, int K, int S) {
  int n, y0, x0;
  const int tk = mie_pick_tile(a.ts, blockIdx.x, n, y0, x0);
  if (tk == 0) return;
  const int co = blockIdx.y * 64 + (threadIdx.x & 63);
  const int pg = threadIdx.x >> 6;
  const int hout = a.ts.h, wout = a.ts.w;
  if (co >= a.cout) return;
  for (int p = 0; p < 16; ++p) {
    const int oy = y0 + 2 * pg + (p >> 3), ox = x0 + (p & 7);
    if (oy >= hout || ox >= wout) continue;
    const long long off = (((long long)n * hout + oy) * wout + ox) * a.cout + co;
    if (tk == 2) { mie_st(a.out, off, 0.f); continue; }
    float acc = 0.f;
    for (int ky = 0; ky < K; ++ky) {
      const int ty = oy + a.pad - ky;
      if (ty < 0 || (ty % S) != 0 || ty / S >= a.h_in) continue;
      for (int kx = 0; kx < K; ++kx) {
        const int tx = ox + a.pad - kx;
        if (tx < 0 || (tx % S) != 0 || tx / S >= a.w_in) continue;
        const long long po = ((long long)n * a.h_in + ty / S) * a.w_in + tx / S;
        if (a.xm != nullptr && !a.xm[po]) continue;
        const T* xr = a.x + po * a.c1;
        const float* wp = a.filt + (long long)(ky * K + kx) * a.cout + co;
        for (int ci = 0; ci < a.c1; ++ci) acc += mie_ld(xr, ci) * wp[(long long)ci * K * K * a.cout];
      }
    }
    conv_store(a, off, co, acc);
  }
}

// The decoder geometry (3x3, stride 2, pad 1, output exactly twice the input) over very few input
// channels -- the 2-channel flow estimate in front of an EVFlowNet decoder, whose result rides into the
// matrix-core transposed conv as its addend.  An output pixel (oy, ox) sees the taps of its sub-pixel
// phase only: ky = 1 for even oy, ky in {0, 2} for odd oy (input row (oy + 1 - ky) / 2), the same in x,
// so 1, 2 or 4 taps -- no division, no modulo.  A thread owns 4 adjacent output channels of one pixel
// (16-byte filter loads, the input values are broadcast loads); the workgroups of grid row x share one
// 8x8 output tile.
template <typename T>
__global__ __launch_bounds__(256) void k_tconv2x_fewcin(ConvArgsT<T> a) {
  int n, y0, x0;
  const int tk = mie_pick_tile(a.ts, blockIdx.x + conv_args_entry_zero(a), n, y0, x0);
  if (tk == 0) return;
  const int hout = a.ts.h, wout = a.ts.w, cout = a.cout, c1 = a.c1;
  const int G = cout >> 2;
  // one (pixel, channel group) per thread: grid y covers the 64 * G items of a tile, so that a tile's
  // dependent loads are one chain deep whatever the channel count
  for (int idx = blockIdx.y * 256 + threadIdx.x; idx < 64 * G; idx += 256 * gridDim.y) {
    const int p = idx / G, g = idx - p * G;
    const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
    if (oy >= hout || ox >= wout) continue;
    const long long off = (((long long)n * hout + oy) * wout + ox) * cout + 4 * g;
    if (tk == 2) {
#pragma unroll
      for (int e = 0; e < 4; ++e) mie_st(a.out, off + e, 0.f);
      continue;
    }
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    const int nky = (oy & 1) ? 2 : 1, nkx = (ox & 1) ? 2 : 1;
    for (int iky = 0; iky < nky; ++iky) {
      const int ky = (oy & 1) ? 2 * iky : 1;
      const int iy = (oy + 1 - ky) >> 1;
      if (iy >= a.h_in) continue;
      for (int ikx = 0; ikx < nkx; ++ikx) {
        const int kx = (ox & 1) ? 2 * ikx : 1;
        const int ix = (ox + 1 - kx) >> 1;
        if (ix >= a.w_in) continue;
        const long long po = ((long long)n * a.h_in + iy) * a.w_in + ix;
        if (a.xm != nullptr && !a.xm[po]) continue;
        const T* xr = a.x + po * c1;
        const float* wp = a.filt + (long long)(ky * 3 + kx) * cout + 4 * g;
        for (int ci = 0; ci < c1; ++ci) {
          const float xv = mie_ld(xr, ci);
          const float4 w4 = *reinterpret_cast<const float4*>(wp + (long long)ci * 9 * cout);
          acc[0] += xv * w4.x; acc[1] += xv * w4.y; acc[2] += xv * w4.z; acc[3] += xv * w4.w;
        }
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) conv_store(a, off + e, 4 * g + e, acc[e]);
  }
}

template <typename T, int K, int S>
void launch_conv(const ConvArgsT<T>& a, unsigned cap, hipStream_t st) {
  if (K == 1 && S == 1 && a.pad == 0 && a.cout <= 4 && (a.c1 & 3) == 0 && (a.c2 & 3) == 0) {
    hipLaunchKernelGGL((k_conv1x1_smallco<T>), dim3(cap), dim3(256), 0, st, a);
  } else if (a.cout <= 4) {
    hipLaunchKernelGGL((k_conv_smallco<T, K, S>), dim3(cap), dim3(64), 0, st, a);
  } else {
    hipLaunchKernelGGL((k_conv_valu<T, K, S>), dim3(cap, mie_div_up(a.cout, 64)), dim3(256), 0, st, a);
  }
}

template <typename T> constexpr int dtype_of() { return sizeof(T) == 4 ? MIE_DTYPE_F32 : MIE_DTYPE_BF16; }

int check_epilogue(const char* who, const void* out_delta, float* reservoir, int act_kind,
                   bool refresh = false) {
  MIE_REQUIRE(out_delta != nullptr, MIE_ERR_INVALID_ARG, "%s: out_delta is NULL", who);
  MIE_REQUIRE(mie_aligned(out_delta, 16) && mie_aligned(reservoir, 16), MIE_ERR_INVALID_ARG,
              "%s: out_delta / reservoir must be 16-byte aligned", who);
  MIE_REQUIRE(act_kind >= MIE_ACT_NONE && act_kind <= MIE_ACT_TANH, MIE_ERR_UNSUPPORTED,
              "%s: unknown activation %d", who, act_kind);
  MIE_REQUIRE(refresh || reservoir != nullptr || act_kind == MIE_ACT_NONE, MIE_ERR_INVALID_ARG,
              "%s: activation %d needs a reservoir", who, act_kind);
  return MIE_OK;
}

// Extra operands of the conv with the ConvLSTM gate chain as its epilogue.
template <typename T>
struct GatesOperands {
  int hid;
  const T* cprev_delta; const uint8_t* cprev_mask; float* cprev_res; float* cell_res;
  T* h_delta; T* c_delta;
};

template <typename T>
int conv_impl(const char* who, const T* x, const uint8_t* xmask, int c1, const T* x2,
              const uint8_t* x2mask, int c2, int h_in, int w_in, const float* filter,
              const T* filter_mc, int cin_total, int k, int stride, int pad, int cout,
              const mie_tileset* out,
              T* out_delta, const T* addend, float* reservoir, int act_kind, float slope,
              int path, bool refresh, const float* bias, void* stream,
              const GatesOperands<T>* gates = nullptr, void* workspace = nullptr,
              long long workspace_bytes = 0, bool x3 = false) {
  mie_clear_error();
  int rc = mie_check_tileset(out, who);
  if (rc != MIE_OK) return rc;
  MIE_REQUIRE(x != nullptr && filter != nullptr, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(c1 > 0 && c2 >= 0 && cout > 0 && cin_total > 0 && h_in > 0 && w_in > 0,
              MIE_ERR_INVALID_ARG, "%s: sizes must be positive (c1=%d c2=%d cout=%d cin=%d h=%d w=%d)",
              who, c1, c2, cout, cin_total, h_in, w_in);
  MIE_REQUIRE((x2 != nullptr) == (c2 > 0), MIE_ERR_INVALID_ARG,
              "%s: x2 and c2 must be given together", who);
  MIE_REQUIRE(x2 != nullptr || x2mask == nullptr, MIE_ERR_INVALID_ARG, "%s: mask of absent x2", who);
  MIE_REQUIRE((long long)c1 + c2 <= cin_total, MIE_ERR_INVALID_ARG,
              "%s: c1 + c2 = %d exceeds the filter's %d input channels", who, c1 + c2, cin_total);
  MIE_REQUIRE(k == 1 || k == 3 || k == 5 || k == 7, MIE_ERR_UNSUPPORTED,
              "%s: kernel size %d not implemented (1, 3, 5, 7)", who, k);
  MIE_REQUIRE(stride == 1 || stride == 2, MIE_ERR_UNSUPPORTED,
              "%s: stride %d not implemented (1, 2)", who, stride);
  MIE_REQUIRE(pad >= 0 && pad <= k, MIE_ERR_INVALID_ARG, "%s: padding %d out of range", who, pad);
  MIE_REQUIRE(h_in + 2 * pad >= k && w_in + 2 * pad >= k, MIE_ERR_INVALID_ARG,
              "%s: input (%d,%d) smaller than the kernel", who, h_in, w_in);
  const int ho = (h_in + 2 * pad - k) / stride + 1, wo = (w_in + 2 * pad - k) / stride + 1;
  MIE_REQUIRE(ho == out->h && wo == out->w, MIE_ERR_INVALID_ARG,
              "%s: conv output is (%d,%d) but the tile set is (%d,%d)", who, ho, wo, out->h, out->w);
  MIE_REQUIRE((long long)out->n * h_in * w_in * (long long)(c1 > c2 ? c1 : c2) < (1LL << 40) &&
                  (long long)out->n * h_in * w_in < 0x7fffffffLL,
              MIE_ERR_CAPACITY, "%s: input too large", who);
  MIE_REQUIRE(mie_aligned(x, 16) && mie_aligned(x2, 16) && mie_aligned(filter, 16),
              MIE_ERR_INVALID_ARG, "%s: x / x2 / filter must be 16-byte aligned", who);
  if (gates == nullptr) {
    rc = check_epilogue(who, out_delta, reservoir, act_kind, refresh);
    if (rc != MIE_OK) return rc;
  }
  MIE_REQUIRE(mie_aligned(bias, 4) && mie_aligned(addend, 16), MIE_ERR_INVALID_ARG,
              "%s: bias must be 4-byte and addend 16-byte aligned", who);
  MIE_REQUIRE(addend == nullptr || addend != out_delta, MIE_ERR_INVALID_ARG,
              "%s: addend must not alias out_delta", who);
  // A workgroup stages the halo of its tile, i.e. pixels that other workgroups of the launch write (their
  // outputs, and the zeros of stale tiles): only a 1x1 conv, which reads no halo, may run in place.
  MIE_REQUIRE(k == 1 || ((const void*)x != (const void*)out_delta && (x2 == nullptr || (const void*)x2 != (const void*)out_delta)),
              MIE_ERR_INVALID_ARG, "%s: x / x2 must not alias out_delta for k > 1", who);
  MIE_REQUIRE(gates == nullptr ||
                  ((const void*)x != (const void*)gates->h_delta && (const void*)x != (const void*)gates->c_delta &&
                   (x2 == nullptr || ((const void*)x2 != (const void*)gates->h_delta &&
                                      (const void*)x2 != (const void*)gates->c_delta))),
              MIE_ERR_INVALID_ARG, "%s: x / x2 must not alias h_delta / c_delta (keep two sets of state buffers "
              "when the state deltas are fed back)", who);
  MIE_REQUIRE((xmask == nullptr || xmask != (const uint8_t*)out->pixmask || k == 1) &&
                  (x2mask == nullptr || x2mask != (const uint8_t*)out->pixmask || k == 1),
              MIE_ERR_INVALID_ARG, "%s: an input mask must not be the output tile set's pixel mask for k > 1", who);
  const int pmul = 32 / (int)sizeof(T);       // input channels per block of the matrix-core filter copy
  MIE_REQUIRE(mie_aligned(filter_mc, 16), MIE_ERR_INVALID_ARG, "%s: filter_mc must be 16-byte aligned", who);
  MIE_REQUIRE(workspace_bytes >= 0 && (workspace != nullptr || workspace_bytes == 0) && mie_aligned(workspace, 16),
              MIE_ERR_INVALID_ARG, "%s: workspace must be 16-byte aligned, with a size >= 0 (0 if NULL)", who);
  MIE_REQUIRE(workspace == nullptr || (workspace != (void*)out_delta && workspace != (void*)reservoir &&
                                       workspace != (const void*)x && workspace != (const void*)x2),
              MIE_ERR_INVALID_ARG, "%s: workspace must not alias an operand", who);
  MIE_REQUIRE(!x3 || (sizeof(T) == 4 && path != MIE_PATH_VALU), MIE_ERR_INVALID_ARG,
              "%s: MIE_DTYPE_F32_BF16X3 is a mode of the matrix-core path for fp32 deltas", who);
  const bool mfma_ok = x3 ? (filter_mc != nullptr && cin_total % 16 == 0 && mie_conv_x3_takes(k, stride, c1, c2, cout))
                          : ((filter_mc != nullptr) && (cin_total % pmul == 0) &&
                             mie_conv_mfma_takes(k, stride, dtype_of<T>(), c1, c2, cout));
  MIE_REQUIRE(!x3 || mfma_ok, MIE_ERR_UNSUPPORTED,
              "%s: MIE_DTYPE_F32_BF16X3 needs filter_mc packed in that layout, k = 3 or 5 and channel counts "
              "in whole chunks (32, stride 2: 16; k=%d stride=%d c1=%d c2=%d cout=%d); see mie_conv_f32x3_takes", who, k, stride,
              c1, c2, cout);
  MIE_REQUIRE(path == MIE_PATH_AUTO || path == MIE_PATH_VALU || path == MIE_PATH_MFMA,
              MIE_ERR_INVALID_ARG, "%s: unknown path %d", who, path);
  MIE_REQUIRE(path != MIE_PATH_MFMA || mfma_ok, MIE_ERR_UNSUPPORTED,
              "%s: MFMA path needs filter_mc (mie_pack_filter) and channel counts in whole staging chunks "
              "and output slabs for k=%d stride=%d (filter_mc=%p c1=%d c2=%d cout=%d)", who, k, stride,
              (const void*)filter_mc, c1, c2, cout);
  const bool auto_path = path == MIE_PATH_AUTO;
  if (path == MIE_PATH_AUTO) path = mfma_ok ? MIE_PATH_MFMA : MIE_PATH_VALU;

  ConvArgsT<T> a;
  a.x = x; a.xm = xmask; a.c1 = c1; a.x2 = x2; a.x2m = x2mask; a.c2 = c2;
  a.h_in = h_in; a.w_in = w_in; a.filt = filter; a.cin_total = cin_total; a.filt_mc = filter_mc;
  a.pad = pad; a.cout = cout; a.out = out_delta; a.res = reservoir; a.act = act_kind;
  a.slope = slope; a.addend = addend; a.refresh = refresh ? 1 : 0; a.bias = bias;
  a.hid = 0; a.g_cpd = nullptr; a.g_cpm = nullptr; a.g_cpres = nullptr; a.g_cres = nullptr;
  a.g_dh = nullptr; a.g_dc = nullptr;
  a.ws = nullptr; a.ws_floats = 0; a.ws_plane = 0; a.xcd_fs = 0; a.x3 = x3 ? 1 : 0;
  a.ts = mie_dev_tileset(out);
  const unsigned cap = (unsigned)mie_tile_capacity(out->n, out->h, out->w);
  hipStream_t st = (hipStream_t)stream;
  if (gates != nullptr) {
    MIE_REQUIRE(mfma_ok && gates->hid % 8 == 0 && cout == 4 * gates->hid, MIE_ERR_UNSUPPORTED,
                "%s: needs filter_mc, whole 32-channel (bf16: 64) input chunks and hid %% 8 == 0 "
                "(c1=%d c2=%d hid=%d)", who, c1, c2, gates->hid);
    a.hid = gates->hid; a.g_cpd = gates->cprev_delta; a.g_cpm = gates->cprev_mask;
    a.g_cpres = gates->cprev_res; a.g_cres = gates->cell_res; a.g_dh = gates->h_delta;
    a.g_dc = gates->c_delta;
    a.ws = (float*)workspace;
    a.ws_floats = workspace_bytes / 4;
    MIE_REQUIRE(mie_launch_conv_gates_mfma(a, cap, st), MIE_ERR_UNSUPPORTED,
                "%s: no kernel variant for cout=%d", who, cout);
    return mie_check_launch(who);
  }
  if (path == MIE_PATH_MFMA) {
    a.ws = (float*)workspace;
    a.ws_floats = workspace_bytes / 4;
    MIE_REQUIRE(mie_launch_conv_mfma(a, k, stride, cap, st), MIE_ERR_UNSUPPORTED,
                "%s: no MFMA kernel variant for k=%d stride=%d cout=%d", who, k, stride, cout);
    return mie_check_launch(who);
  }
  // very few input channels (network heads): a matrix-core kernel of its own, unless the VALU path was asked for
  if (auto_path && mie_launch_conv_fewcin(a, k, stride, cap, st)) return mie_check_launch(who);
  switch (k * 10 + stride) {
    case 11: launch_conv<T, 1, 1>(a, cap, st); break;
    case 12: launch_conv<T, 1, 2>(a, cap, st); break;
    case 31: launch_conv<T, 3, 1>(a, cap, st); break;
    case 32: launch_conv<T, 3, 2>(a, cap, st); break;
    case 51: launch_conv<T, 5, 1>(a, cap, st); break;
    case 52: launch_conv<T, 5, 2>(a, cap, st); break;
    case 71: launch_conv<T, 7, 1>(a, cap, st); break;
    case 72: launch_conv<T, 7, 2>(a, cap, st); break;
    default: MIE_REQUIRE(false, MIE_ERR_UNSUPPORTED, "%s: k=%d stride=%d", who, k, stride);
  }
  return mie_check_launch(who);
}

}  // namespace

// P[ci/B][tap][(ci%B)/(B/2)][co][ci%(B/2)] = F[ci][tap][co], B = 8 (fp32) or 16 (bf16) input
// channels per block: the k-steps one MFMA lane multiplies for a tap are 16 contiguous bytes.
template <typename T>
__global__ __launch_bounds__(256) void k_pack_filter(const float* __restrict__ f, T* __restrict__ p,
                                                     int cin, int kk, int cout) {
  constexpr int B = 32 / (int)sizeof(T), HB = B / 2;
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long total = (long long)cin * kk * cout;
  if (i >= total) return;
  const int co = (int)(i % cout);
  const long long t = i / cout;
  const int tap = (int)(t % kk);
  const int ci = (int)(t / kk);
  const long long o = ((((long long)(ci / B) * kk + tap) * 2 + (ci % B) / HB) * cout + co) * HB + (ci % HB);
  mie_st(p, o, f[i]);
}

// The three-term copy for MIE_DTYPE_F32_BF16X3: every weight as hi + mid + lo in bf16 (each rounded to nearest even),
// P[ci/16][tap][term][(ci%16)/8][co][ci%8].
__global__ __launch_bounds__(256) void k_pack_filter_x3(const float* __restrict__ f, mie_bf16* __restrict__ p,
                                                        int cin, int kk, int cout) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long total = (long long)cin * kk * cout;
  if (i >= total) return;
  const int co = (int)(i % cout);
  const long long t = i / cout;
  const int tap = (int)(t % kk);
  const int ci = (int)(t / kk);
  const float v = f[i];
  const mie_bf16 hi = (mie_bf16)v;
  const float r1 = v - (float)hi;
  const mie_bf16 mid = (mie_bf16)r1;
  const mie_bf16 lo = (mie_bf16)(r1 - (float)mid);
  const long long o = (((((long long)(ci / 16) * kk + tap) * 3) * 2 + (ci % 16) / 8) * cout + co) * 8 + (ci % 8);
  const long long term = 2LL * cout * 8;
  p[o] = hi;
  p[o + term] = mid;
  p[o + 2 * term] = lo;
}

namespace {

template <typename T>
int tconv_impl(const char* who, const T* x, const uint8_t* xmask, int cin, int h_in, int w_in,
               const float* filter, int k, int stride, int pad, int cout, const mie_tileset* out,
               T* out_delta, float* reservoir, int act_kind, float slope, bool refresh,
               const float* bias, void* stream) {
  ConvArgsT<T> a;
  a.x = x; a.xm = xmask; a.c1 = cin; a.x2 = nullptr; a.x2m = nullptr; a.c2 = 0;
  a.h_in = h_in; a.w_in = w_in; a.filt = filter; a.cin_total = cin; a.filt_mc = nullptr;
  a.pad = pad; a.cout = cout; a.out = out_delta; a.res = reservoir; a.act = act_kind;
  a.slope = slope; a.addend = nullptr; a.refresh = refresh ? 1 : 0; a.bias = bias;
  a.hid = 0; a.g_cpd = nullptr; a.g_cpm = nullptr; a.g_cpres = nullptr; a.g_cres = nullptr;
  a.g_dh = nullptr; a.g_dc = nullptr;
  a.ws = nullptr; a.ws_floats = 0; a.ws_plane = 0; a.xcd_fs = 0; a.x3 = 0;
  a.ts = mie_dev_tileset(out);
  const unsigned cap = (unsigned)mie_tile_capacity(out->n, out->h, out->w);
  if (k == 3 && stride == 2 && pad == 1 && out->h == 2 * h_in && out->w == 2 * w_in && cin <= 8 && cout % 4 == 0 &&
      mie_aligned(filter, 16))
    hipLaunchKernelGGL(k_tconv2x_fewcin<T>, dim3(cap, mie_div_up(16 * cout, 256)), dim3(256), 0, (hipStream_t)stream, a);
  else
    hipLaunchKernelGGL(k_tconv_valu<T>, dim3(cap, mie_div_up(cout, 64)), dim3(256), 0,
                       (hipStream_t)stream, a, k, stride);
  return mie_check_launch(who);
}

}  // namespace

#define MIE_CONV_DTYPE_OK(dtype, who)                                                     \
  do {                                                                                    \
    mie_clear_error();                                                                    \
    MIE_REQUIRE((dtype) == MIE_DTYPE_F32 || (dtype) == MIE_DTYPE_BF16, MIE_ERR_UNSUPPORTED, \
                "%s: unknown delta dtype %d", who, (int)(dtype));                         \
  } while (0)
// The entry points of the matrix-core conv also take MIE_DTYPE_F32_BF16X3: fp32 deltas, three-term filter copy.
#define MIE_CONV_DTYPE_X3_OK(dtype, who, x3)                                              \
  do {                                                                                    \
    if ((dtype) == MIE_DTYPE_F32_BF16X3) {                                                \
      x3 = true;                                                                          \
      dtype = MIE_DTYPE_F32;                                                              \
    }                                                                                     \
    MIE_CONV_DTYPE_OK(dtype, who);                                                        \
  } while (0)

extern "C" int mie_conv_f32x3_takes(int k, int stride, int c1, int c2, int cout) {
  return mie_conv_x3_takes(k, stride, c1, c2, cout) ? 1 : 0;
}

extern "C" int mie_pack_filter(const float* filter, int cin, int k, int cout, void* packed,
                               int dtype, void* stream) {
  const char* who = "mie_pack_filter";
  bool x3 = false;
  MIE_CONV_DTYPE_X3_OK(dtype, who, x3);
  MIE_REQUIRE(filter && packed, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(cin > 0 && k > 0 && cout > 0, MIE_ERR_INVALID_ARG, "%s: sizes must be positive", who);
  const int blk = (dtype == MIE_DTYPE_BF16 || x3) ? 16 : 8;
  MIE_REQUIRE(cin % blk == 0, MIE_ERR_UNSUPPORTED, "%s: cin = %d is not a multiple of %d", who, cin, blk);
  MIE_REQUIRE(mie_aligned(filter, 16) && mie_aligned(packed, 16) && (const void*)filter != packed,
              MIE_ERR_INVALID_ARG, "%s: buffers must be 16-byte aligned and distinct", who);
  const long long total = (long long)cin * k * k * cout;
  MIE_REQUIRE(total < (1LL << 40), MIE_ERR_CAPACITY, "%s: filter too large", who);
  const dim3 grid((unsigned)((total + 255) / 256));
  if (x3)
    hipLaunchKernelGGL(k_pack_filter_x3, grid, dim3(256), 0, (hipStream_t)stream, filter, (mie_bf16*)packed, cin,
                       k * k, cout);
  else if (dtype == MIE_DTYPE_BF16)
    hipLaunchKernelGGL(k_pack_filter<mie_bf16>, grid, dim3(256), 0, (hipStream_t)stream, filter,
                       (mie_bf16*)packed, cin, k * k, cout);
  else
    hipLaunchKernelGGL(k_pack_filter<float>, grid, dim3(256), 0, (hipStream_t)stream, filter,
                       (float*)packed, cin, k * k, cout);
  return mie_check_launch(who);
}

extern "C" int mie_conv_masked(const void* x, const uint8_t* xmask, int c1, const void* x2,
                               const uint8_t* x2mask, int c2, int h_in, int w_in,
                               const float* filter, const void* filter_mc, int cin_total, int k,
                               int stride, int pad, int cout, const mie_tileset* out,
                               void* out_delta, const void* addend, float* reservoir,
                               int act_kind, float slope, int path, int dtype, void* stream) {
  const char* who = "mie_conv_masked";
  bool x3 = false;
  MIE_CONV_DTYPE_X3_OK(dtype, who, x3);
  if (dtype == MIE_DTYPE_BF16) {
    typedef mie_bf16 T;
    return conv_impl<T>(who, (const T*)x, xmask, c1, (const T*)x2, x2mask, c2, h_in, w_in, filter,
                        (const T*)filter_mc, cin_total, k, stride, pad, cout, out, (T*)out_delta,
                        (const T*)addend, reservoir, act_kind, slope, path, false, nullptr, stream);
  }
  typedef float T;
  return conv_impl<T>(who, (const T*)x, xmask, c1, (const T*)x2, x2mask, c2, h_in, w_in, filter,
                      (const T*)filter_mc, cin_total, k, stride, pad, cout, out, (T*)out_delta,
                      (const T*)addend, reservoir, act_kind, slope, path, false, nullptr, stream, nullptr, nullptr, 0, x3);
}

extern "C" int mie_conv_masked_ws(const void* x, const uint8_t* xmask, int c1, const void* x2,
                                  const uint8_t* x2mask, int c2, int h_in, int w_in,
                                  const float* filter, const void* filter_mc, int cin_total, int k,
                                  int stride, int pad, int cout, const mie_tileset* out,
                                  void* out_delta, const void* addend, float* reservoir,
                                  int act_kind, float slope, int path, int dtype, void* workspace,
                                  long long workspace_bytes, void* stream) {
  const char* who = "mie_conv_masked_ws";
  bool x3 = false;
  MIE_CONV_DTYPE_X3_OK(dtype, who, x3);
  if (dtype == MIE_DTYPE_BF16) {
    typedef mie_bf16 T;
    return conv_impl<T>(who, (const T*)x, xmask, c1, (const T*)x2, x2mask, c2, h_in, w_in, filter,
                        (const T*)filter_mc, cin_total, k, stride, pad, cout, out, (T*)out_delta,
                        (const T*)addend, reservoir, act_kind, slope, path, false, nullptr, stream, nullptr,
                        workspace, workspace_bytes);
  }
  typedef float T;
  return conv_impl<T>(who, (const T*)x, xmask, c1, (const T*)x2, x2mask, c2, h_in, w_in, filter,
                      (const T*)filter_mc, cin_total, k, stride, pad, cout, out, (T*)out_delta,
                      (const T*)addend, reservoir, act_kind, slope, path, false, nullptr, stream, nullptr,
                      workspace, workspace_bytes, x3);
}

// ---- the workspace form for callers that cannot allocate ---------------------------------------
// The split form's partial sums live in a device-resident array instead of a caller workspace.  The
// array's name is only a host-side handle: its device address differs per GPU and is looked up once
// per device (with that device current) on the entry point's first call there; kernels and every
// other use take that address.
#define MIE_NOALLOC_MAX_DEVICES 64
static __device__ __align__(256) float scratch[MIE_NOALLOC_WS_BYTES / 4];

namespace {
int noalloc_scratch(const char* who, float** out) {
  static float* ptrs[MIE_NOALLOC_MAX_DEVICES];      // zero-initialised; written once per device
  static bool known[MIE_NOALLOC_MAX_DEVICES];
  static std::mutex mu;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  MIE_REQUIRE(e == hipSuccess && dev >= 0 && dev < MIE_NOALLOC_MAX_DEVICES, MIE_ERR_LAUNCH,
              "%s: no current device (%s)", who, hipGetErrorString(e));
  std::lock_guard<std::mutex> lock(mu);
  if (!known[dev]) {
    float* p = nullptr;
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
    MIE_REQUIRE(e == hipSuccess && p != nullptr, MIE_ERR_LAUNCH,
                "%s: the device-resident workspace has no address on device %d (%s)", who, dev,
                hipGetErrorString(e));
    ptrs[dev] = p;
    known[dev] = true;
  }
  *out = ptrs[dev];
  return MIE_OK;
}
}  // namespace

extern "C" int mie_conv_masked_noalloc(const void* x, const uint8_t* xmask, int c1, const void* x2,
                                       const uint8_t* x2mask, int c2, int h_in, int w_in,
                                       const float* filter, const void* filter_mc, int cin_total, int k,
                                       int stride, int pad, int cout, const mie_tileset* out,
                                       void* out_delta, const void* addend, float* reservoir,
                                       int act_kind, float slope, int path, int dtype, void* stream) {
  const char* who = "mie_conv_masked_noalloc";
  bool x3 = false;
  MIE_CONV_DTYPE_X3_OK(dtype, who, x3);
  int rc = mie_check_tileset(out, who);
  if (rc != MIE_OK) return rc;
  MIE_REQUIRE(cout > 0, MIE_ERR_INVALID_ARG, "%s: cout must be positive", who);
  // two partial planes of the output must fit: beyond that the launch is no "plane of very few tiles"
  const long long plane_bytes = (long long)out->n * out->h * out->w * cout * 4;
  MIE_REQUIRE(2 * plane_bytes <= (long long)MIE_NOALLOC_WS_BYTES, MIE_ERR_CAPACITY,
              "%s: an output plane of %lld bytes (n=%d h=%d w=%d cout=%d) exceeds the device-resident "
              "workspace, which holds two planes of at most %lld bytes each; use mie_conv_masked for "
              "larger outputs", who, plane_bytes, out->n, out->h, out->w, cout,
              (long long)MIE_NOALLOC_WS_BYTES / 2);
  float* ws = nullptr;
  rc = noalloc_scratch(who, &ws);
  if (rc != MIE_OK) return rc;
  if (dtype == MIE_DTYPE_BF16) {
    typedef mie_bf16 T;
    return conv_impl<T>(who, (const T*)x, xmask, c1, (const T*)x2, x2mask, c2, h_in, w_in, filter,
                        (const T*)filter_mc, cin_total, k, stride, pad, cout, out, (T*)out_delta,
                        (const T*)addend, reservoir, act_kind, slope, path, false, nullptr, stream, nullptr,
                        ws, (long long)MIE_NOALLOC_WS_BYTES);
  }
  typedef float T;
  return conv_impl<T>(who, (const T*)x, xmask, c1, (const T*)x2, x2mask, c2, h_in, w_in, filter,
                      (const T*)filter_mc, cin_total, k, stride, pad, cout, out, (T*)out_delta,
                      (const T*)addend, reservoir, act_kind, slope, path, false, nullptr, stream, nullptr,
                      ws, (long long)MIE_NOALLOC_WS_BYTES, x3);
}

extern "C" int mie_conv_refresh(const void* x, int c1, const void* x2, int c2, int h_in,
                                int w_in, const float* filter, const void* filter_mc,
                                int cin_total, int k, int stride, int pad, int cout,
                                const float* bias, const mie_tileset* out,
                                void* out_dense, const void* addend, float* reservoir,
                                int act_kind, float slope, int path, int dtype, void* stream) {
  const char* who = "mie_conv_refresh";
  bool x3 = false;
  MIE_CONV_DTYPE_X3_OK(dtype, who, x3);
  if (dtype == MIE_DTYPE_BF16) {
    typedef mie_bf16 T;
    return conv_impl<T>(who, (const T*)x, nullptr, c1, (const T*)x2, nullptr, c2, h_in, w_in, filter,
                        (const T*)filter_mc, cin_total, k, stride, pad, cout, out, (T*)out_dense,
                        (const T*)addend, reservoir, act_kind, slope, path, true, bias, stream);
  }
  typedef float T;
  return conv_impl<T>(who, (const T*)x, nullptr, c1, (const T*)x2, nullptr, c2, h_in, w_in, filter,
                      (const T*)filter_mc, cin_total, k, stride, pad, cout, out, (T*)out_dense,
                      (const T*)addend, reservoir, act_kind, slope, path, true, bias, stream, nullptr, nullptr, 0, x3);
}

namespace {
template <typename T>
int conv_gates_entry(const char* who, const void* x, const uint8_t* xmask, int c1, const void* x2,
                     const uint8_t* x2mask, int c2, int h_in, int w_in, const float* filter,
                     const void* filter_mc, int cin_total, int hid, const mie_tileset* out,
                     float* gates_res, const void* cprev_delta, const uint8_t* cprev_mask,
                     float* cprev_res, float* cell_res, void* h_delta, void* c_delta, void* workspace,
                     long long workspace_bytes, void* stream, bool x3 = false) {
  MIE_REQUIRE(hid > 0 && hid <= (1 << 20), MIE_ERR_INVALID_ARG, "%s: hid = %d out of range", who, hid);
  MIE_REQUIRE(gates_res && cprev_res && cell_res && h_delta && c_delta, MIE_ERR_INVALID_ARG,
              "%s: NULL pointer", who);
  MIE_REQUIRE(cprev_delta != nullptr || cprev_mask == nullptr, MIE_ERR_INVALID_ARG,
              "%s: mask of absent cprev_delta", who);
  MIE_REQUIRE(mie_aligned(gates_res, 16) && mie_aligned(cprev_delta, 16) && mie_aligned(cprev_res, 16) &&
                  mie_aligned(cell_res, 16) && mie_aligned(h_delta, 16) && mie_aligned(c_delta, 16),
              MIE_ERR_INVALID_ARG, "%s: buffers must be 16-byte aligned", who);
  GatesOperands<T> g;
  g.hid = hid; g.cprev_delta = (const T*)cprev_delta; g.cprev_mask = cprev_mask; g.cprev_res = cprev_res;
  g.cell_res = cell_res; g.h_delta = (T*)h_delta; g.c_delta = (T*)c_delta;
  return conv_impl<T>(who, (const T*)x, xmask, c1, (const T*)x2, x2mask, c2, h_in, w_in, filter,
                      (const T*)filter_mc, cin_total, 3, 1, 1, 4 * hid, out, (T*)nullptr, (const T*)nullptr,
                      gates_res, MIE_ACT_NONE, 0.f, MIE_PATH_MFMA, false, nullptr, stream, &g, workspace, workspace_bytes, x3);
}

int tconv_entry(const char* who, const void* x, const uint8_t* xmask, int cin, int h_in, int w_in,
                const float* filter, int k, int stride, int pad, int cout, const mie_tileset* out,
                void* out_delta, float* reservoir, int act_kind, float slope, bool refresh,
                const float* bias, int dtype, void* stream) {
  MIE_CONV_DTYPE_OK(dtype, who);
  int rc = mie_check_tileset(out, who);
  if (rc != MIE_OK) return rc;
  MIE_REQUIRE(x != nullptr && filter != nullptr, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(cin > 0 && cout > 0 && h_in > 0 && w_in > 0, MIE_ERR_INVALID_ARG,
              "%s: sizes must be positive", who);
  MIE_REQUIRE(k >= 1 && k <= 7 && stride >= 1 && stride <= 4 && pad >= 0 && pad < k,
              MIE_ERR_UNSUPPORTED, "%s: k=%d stride=%d pad=%d not implemented", who, k, stride, pad);
  const int hmin = (h_in - 1) * stride - 2 * pad + k, wmin = (w_in - 1) * stride - 2 * pad + k;
  MIE_REQUIRE(out->h >= hmin && out->h < hmin + stride && out->w >= wmin && out->w < wmin + stride,
              MIE_ERR_INVALID_ARG, "%s: output (%d,%d) not in [(%d,%d), +stride)", who, out->h,
              out->w, hmin, wmin);
  MIE_REQUIRE((long long)out->n * h_in * w_in < 0x7fffffffLL, MIE_ERR_CAPACITY,
              "%s: input too large", who);
  MIE_REQUIRE(mie_aligned(x, 16) && mie_aligned(filter, 16) && mie_aligned(bias, 4), MIE_ERR_INVALID_ARG,
              "%s: x / filter must be 16-byte, bias 4-byte aligned", who);
  rc = check_epilogue(who, out_delta, reservoir, act_kind, refresh);
  if (rc != MIE_OK) return rc;
  if (dtype == MIE_DTYPE_BF16)
    return tconv_impl<mie_bf16>(who, (const mie_bf16*)x, xmask, cin, h_in, w_in, filter, k, stride, pad,
                                cout, out, (mie_bf16*)out_delta, reservoir, act_kind, slope, refresh, bias,
                                stream);
  return tconv_impl<float>(who, (const float*)x, xmask, cin, h_in, w_in, filter, k, stride, pad, cout,
                           out, (float*)out_delta, reservoir, act_kind, slope, refresh, bias, stream);
}
}  // namespace

extern "C" int mie_tconv_masked(const void* x, const uint8_t* xmask, int cin, int h_in,
                                int w_in, const float* filter, int k, int stride, int pad,
                                int cout, const mie_tileset* out, void* out_delta,
                                float* reservoir, int act_kind, float slope, int dtype, void* stream) {
  return tconv_entry("mie_tconv_masked", x, xmask, cin, h_in, w_in, filter, k, stride, pad, cout, out,
                     out_delta, reservoir, act_kind, slope, false, nullptr, dtype, stream);
}

extern "C" int mie_tconv_refresh(const void* x, int cin, int h_in, int w_in, const float* filter,
                                 int k, int stride, int pad, int cout, const float* bias,
                                 const mie_tileset* out, void* out_dense, float* reservoir,
                                 int act_kind, float slope, int dtype, void* stream) {
  return tconv_entry("mie_tconv_refresh", x, nullptr, cin, h_in, w_in, filter, k, stride, pad, cout, out,
                     out_dense, reservoir, act_kind, slope, true, bias, dtype, stream);
}

namespace {
template <typename T>
int upconv_entry(const char* who, const void* a_lo, const uint8_t* amask, const void* b_lo, const uint8_t* bmask,
                 int c, int h_lo, int w_lo, const float* filter, const void* filter_mc, int cin_total, int k,
                 int pad, int cout, const mie_tileset* out, void* out_delta, const void* addend, float* reservoir,
                 int act_kind, float slope, void* workspace, long long workspace_bytes, void* stream, bool x3 = false) {
  int rc = mie_check_tileset(out, who);
  if (rc != MIE_OK) return rc;
  MIE_REQUIRE(a_lo && filter, MIE_ERR_INVALID_ARG, "%s: NULL pointer (a and filter are required)", who);
  MIE_REQUIRE(b_lo != nullptr || bmask == nullptr, MIE_ERR_INVALID_ARG, "%s: mask of absent b", who);
  MIE_REQUIRE(c > 0 && cout > 0 && h_lo > 0 && w_lo > 0 && cin_total >= c, MIE_ERR_INVALID_ARG,
              "%s: sizes out of range (c=%d cout=%d cin_total=%d h=%d w=%d)", who, c, cout, cin_total, h_lo, w_lo);
  // a single input of at most 8 channels (the flow estimate in front of an EVFlowNet decoder): 3x3 or 5x5
  const bool few = c <= 8 && b_lo == nullptr && (k == 3 || k == 5) && pad == k / 2 && cout % 32 == 0;
  if (!few) {
    MIE_REQUIRE(k == 5 && pad == 2, MIE_ERR_UNSUPPORTED,
                "%s: only the 5x5 pad-2 conv is implemented for more than 8 channels or two inputs (k=%d pad=%d)", who, k, pad);
    MIE_REQUIRE(filter_mc != nullptr, MIE_ERR_INVALID_ARG, "%s: filter_mc is required", who);
    const int chunk = 128 / (int)sizeof(T);      // 32 fp32 / 64 bf16 channels per staged chunk
    MIE_REQUIRE(c % chunk == 0 && cout % 32 == 0 && cin_total % (x3 ? 16 : 32 / (int)sizeof(T)) == 0, MIE_ERR_UNSUPPORTED,
                "%s: needs c %% %d == 0 and cout %% 32 == 0 (c=%d cout=%d)", who, chunk, c, cout);
  }
  MIE_REQUIRE(out->h == 2 * h_lo && out->w == 2 * w_lo, MIE_ERR_INVALID_ARG,
              "%s: the tile set is (%d,%d), twice the input is (%d,%d)", who, out->h, out->w, 2 * h_lo, 2 * w_lo);
  MIE_REQUIRE((long long)out->n * h_lo * w_lo * c < (1LL << 40) && (long long)out->n * out->h * out->w < 0x7fffffffLL,
              MIE_ERR_CAPACITY, "%s: input too large", who);
  MIE_REQUIRE(mie_aligned(a_lo, 16) && mie_aligned(b_lo, 16) && mie_aligned(filter, 16) && mie_aligned(filter_mc, 16) &&
                  mie_aligned(addend, 16),
              MIE_ERR_INVALID_ARG, "%s: a / b / filter / filter_mc / addend must be 16-byte aligned", who);
  MIE_REQUIRE(addend == nullptr || addend != out_delta, MIE_ERR_INVALID_ARG, "%s: addend must not alias out_delta", who);
  MIE_REQUIRE(workspace_bytes >= 0 && (workspace != nullptr || workspace_bytes == 0) && mie_aligned(workspace, 16),
              MIE_ERR_INVALID_ARG, "%s: workspace must be 16-byte aligned, with a size >= 0 (0 if NULL)", who);
  MIE_REQUIRE(workspace == nullptr || (workspace != out_delta && workspace != (void*)reservoir && workspace != a_lo &&
                                       workspace != b_lo && workspace != addend),
              MIE_ERR_INVALID_ARG, "%s: workspace must not alias an operand", who);
  rc = check_epilogue(who, out_delta, reservoir, act_kind, false);
  if (rc != MIE_OK) return rc;
  ConvArgsT<T> a;
  a.x = (const T*)a_lo; a.xm = amask; a.c1 = c; a.x2 = (const T*)b_lo; a.x2m = bmask; a.c2 = b_lo ? c : 0;
  a.h_in = 2 * h_lo; a.w_in = 2 * w_lo; a.filt = filter; a.cin_total = cin_total; a.filt_mc = (const T*)filter_mc;
  a.pad = pad; a.cout = cout; a.out = (T*)out_delta; a.res = reservoir; a.act = act_kind;
  a.slope = slope; a.addend = (const T*)addend; a.refresh = 0; a.bias = nullptr;
  a.hid = 0; a.g_cpd = nullptr; a.g_cpm = nullptr; a.g_cpres = nullptr; a.g_cres = nullptr;
  a.g_dh = nullptr; a.g_dc = nullptr;
  a.ws = few ? nullptr : (float*)workspace; a.ws_floats = few ? 0 : workspace_bytes / 4; a.ws_plane = 0; a.xcd_fs = 0;
  a.x3 = (x3 && !few) ? 1 : 0;
  a.ts = mie_dev_tileset(out);
  const unsigned cap = (unsigned)mie_tile_capacity(out->n, out->h, out->w);
  if (few) {
    MIE_REQUIRE(mie_launch_conv_fewcin_up(a, k, cap, (hipStream_t)stream), MIE_ERR_UNSUPPORTED,
                "%s: no kernel variant for c=%d cout=%d k=%d", who, c, cout, k);
    return mie_check_launch(who);
  }
  MIE_REQUIRE(mie_launch_conv_up_mfma(a, cap, (hipStream_t)stream), MIE_ERR_UNSUPPORTED,
              "%s: no kernel variant for c=%d cout=%d", who, c, cout);
  return mie_check_launch(who);
}
}  // namespace

extern "C" int mie_upconv_masked_ws(const void* a, const uint8_t* amask, const void* b, const uint8_t* bmask, int c,
                                    int h_in, int w_in, const float* filter, const void* filter_mc, int cin_total,
                                    int k, int pad, int cout, const mie_tileset* out, void* out_delta,
                                    const void* addend, float* reservoir, int act_kind, float slope, int dtype,
                                    void* workspace, long long workspace_bytes, void* stream) {
  const char* who = "mie_upconv_masked";
  bool x3 = false;
  MIE_CONV_DTYPE_X3_OK(dtype, who, x3);
  if (dtype == MIE_DTYPE_BF16)
    return upconv_entry<mie_bf16>(who, a, amask, b, bmask, c, h_in, w_in, filter, filter_mc, cin_total, k, pad, cout,
                                  out, out_delta, addend, reservoir, act_kind, slope, workspace, workspace_bytes, stream);
  return upconv_entry<float>(who, a, amask, b, bmask, c, h_in, w_in, filter, filter_mc, cin_total, k, pad, cout, out,
                             out_delta, addend, reservoir, act_kind, slope, workspace, workspace_bytes, stream, x3);
}

extern "C" int mie_upconv_masked(const void* a, const uint8_t* amask, const void* b, const uint8_t* bmask, int c,
                                 int h_in, int w_in, const float* filter, const void* filter_mc, int cin_total,
                                 int k, int pad, int cout, const mie_tileset* out, void* out_delta,
                                 const void* addend, float* reservoir, int act_kind, float slope, int dtype,
                                 void* stream) {
  return mie_upconv_masked_ws(a, amask, b, bmask, c, h_in, w_in, filter, filter_mc, cin_total, k, pad, cout, out,
                              out_delta, addend, reservoir, act_kind, slope, dtype, nullptr, 0, stream);
}

extern "C" int mie_upconv_pred_masked(const void* a_lo, const uint8_t* amask, const void* b_lo, const uint8_t* bmask,
                                      int c, int h_in, int w_in, const float* filter, const void* filter_mc,
                                      int cin_total, int cout, const mie_tileset* out, float* reservoir, int act_kind,
                                      float slope, const void* skip, const uint8_t* skip_mask, const float* pred_filter,
                                      float* pred_reservoir, int pred_act, float pred_slope, void* pred_delta,
                                      int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_upconv_pred_masked";
  int rc = mie_check_tileset(out, who);
  if (rc != MIE_OK) return rc;
  MIE_REQUIRE(dtype == MIE_DTYPE_BF16 && c == 64 && cout == 32, MIE_ERR_UNSUPPORTED,
              "%s: implemented for bf16 deltas, 64 -> 32 channels (dtype=%d c=%d cout=%d)", who, dtype, c, cout);
  MIE_REQUIRE(a_lo && filter && filter_mc && reservoir && skip && pred_filter && pred_reservoir && pred_delta,
              MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(b_lo != nullptr || bmask == nullptr, MIE_ERR_INVALID_ARG, "%s: mask of absent b", who);
  MIE_REQUIRE(h_in > 0 && w_in > 0 && cin_total >= c && cin_total % 16 == 0, MIE_ERR_INVALID_ARG,
              "%s: sizes out of range (cin_total=%d h=%d w=%d)", who, cin_total, h_in, w_in);
  MIE_REQUIRE(out->h == 2 * h_in && out->w == 2 * w_in, MIE_ERR_INVALID_ARG,
              "%s: the tile set is (%d,%d), twice the input is (%d,%d)", who, out->h, out->w, 2 * h_in, 2 * w_in);
  MIE_REQUIRE((long long)out->n * out->h * out->w < 0x7fffffffLL, MIE_ERR_CAPACITY, "%s: input too large", who);
  MIE_REQUIRE(mie_aligned(a_lo, 16) && mie_aligned(b_lo, 16) && mie_aligned(filter, 16) && mie_aligned(filter_mc, 16) &&
                  mie_aligned(reservoir, 16) && mie_aligned(skip, 16) && mie_aligned(pred_filter, 16) &&
                  mie_aligned(pred_reservoir, 4) && mie_aligned(pred_delta, 2),
              MIE_ERR_INVALID_ARG, "%s: misaligned operand", who);
  MIE_REQUIRE((act_kind == MIE_ACT_NONE || act_kind == MIE_ACT_RELU || act_kind == MIE_ACT_LEAKY_RELU) &&
                  pred_act >= MIE_ACT_NONE && pred_act <= MIE_ACT_TANH,
              MIE_ERR_UNSUPPORTED, "%s: activation %d / %d not implemented", who, act_kind, pred_act);
  MIE_REQUIRE(pred_delta != skip && pred_delta != a_lo && pred_delta != b_lo && (void*)pred_reservoir != (void*)reservoir,
              MIE_ERR_INVALID_ARG, "%s: outputs must not alias inputs", who);
  ConvArgsT<mie_bf16> a;
  a.x = (const mie_bf16*)a_lo; a.xm = amask; a.c1 = c; a.x2 = (const mie_bf16*)b_lo; a.x2m = bmask; a.c2 = b_lo ? c : 0;
  a.h_in = 2 * h_in; a.w_in = 2 * w_in; a.filt = filter; a.cin_total = cin_total; a.filt_mc = (const mie_bf16*)filter_mc;
  a.pad = 2; a.cout = cout; a.out = nullptr; a.res = reservoir; a.act = act_kind;
  a.slope = slope; a.addend = nullptr; a.refresh = 0; a.bias = nullptr;
  a.hid = 0; a.g_cpd = nullptr; a.g_cpm = nullptr; a.g_cpres = nullptr; a.g_cres = nullptr;
  a.g_dh = nullptr; a.g_dc = nullptr;
  a.ws = nullptr; a.ws_floats = 0; a.ws_plane = 0; a.xcd_fs = 0; a.x3 = 0;
  a.ts = mie_dev_tileset(out);
  const unsigned cap = (unsigned)mie_tile_capacity(out->n, out->h, out->w);
  MIE_REQUIRE(mie_launch_upconv_pred_persist(a, (const mie_bf16*)skip, skip_mask, pred_filter, pred_reservoir,
                                             (mie_bf16*)pred_delta, pred_act, pred_slope, cap, (hipStream_t)stream),
              MIE_ERR_UNSUPPORTED, "%s: planes of fewer than 2048 tiles (or more than 2^20) take the separate kernels", who);
  return mie_check_launch(who);
}

extern "C" int mie_conv_gates_masked_ws(const void* x, const uint8_t* xmask, int c1, const void* x2,
                                        const uint8_t* x2mask, int c2, int h_in, int w_in,
                                        const float* filter, const void* filter_mc, int cin_total,
                                        int hid, const mie_tileset* out, float* gates_res,
                                        const void* cprev_delta, const uint8_t* cprev_mask,
                                        float* cprev_res, float* cell_res, void* h_delta,
                                        void* c_delta, int dtype, void* workspace, long long workspace_bytes,
                                        void* stream) {
  const char* who = "mie_conv_gates_masked";
  bool x3 = false;
  MIE_CONV_DTYPE_X3_OK(dtype, who, x3);
  MIE_REQUIRE(workspace == nullptr || (workspace != (void*)gates_res && workspace != (void*)cprev_res && workspace != (void*)cell_res &&
                                       workspace != h_delta && workspace != c_delta && workspace != cprev_delta),
              MIE_ERR_INVALID_ARG, "%s: workspace must not alias an operand", who);
  if (dtype == MIE_DTYPE_BF16)
    return conv_gates_entry<mie_bf16>(who, x, xmask, c1, x2, x2mask, c2, h_in, w_in, filter, filter_mc,
                                      cin_total, hid, out, gates_res, cprev_delta, cprev_mask, cprev_res,
                                      cell_res, h_delta, c_delta, workspace, workspace_bytes, stream);
  return conv_gates_entry<float>(who, x, xmask, c1, x2, x2mask, c2, h_in, w_in, filter, filter_mc, cin_total,
                                 hid, out, gates_res, cprev_delta, cprev_mask, cprev_res, cell_res, h_delta,
                                 c_delta, workspace, workspace_bytes, stream, x3);
}

extern "C" int mie_conv_gates_masked(const void* x, const uint8_t* xmask, int c1, const void* x2,
                                     const uint8_t* x2mask, int c2, int h_in, int w_in,
                                     const float* filter, const void* filter_mc, int cin_total,
                                     int hid, const mie_tileset* out, float* gates_res,
                                     const void* cprev_delta, const uint8_t* cprev_mask,
                                     float* cprev_res, float* cell_res, void* h_delta,
                                     void* c_delta, int dtype, void* stream) {
  return mie_conv_gates_masked_ws(x, xmask, c1, x2, x2mask, c2, h_in, w_in, filter, filter_mc, cin_total, hid, out,
                                  gates_res, cprev_delta, cprev_mask, cprev_res, cell_res, h_delta, c_delta, dtype,
                                  nullptr, 0, stream);
}
