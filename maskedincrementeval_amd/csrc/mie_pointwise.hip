// Point-wise incremental kernels over active tiles (gfx950): activation
// increment, product rule, sum, bilinear x2 up-sampling and the fused ConvLSTM
// gate chain.  All of them are HBM-bound: one 256-thread block walks the
// 64 pixels x C channels of one 8x8 tile with consecutive lanes on consecutive
// channels of the NHWC row (float4 when C % 4 == 0), so a wave reads whole
// 8-pixel rows of the tile as contiguous segments.
#include "mie_common.h"
#include "mie_conv.h"

namespace {

template <int VEC> struct Vec;
template <> struct Vec<4> {
  float4 v;
  __device__ static Vec load(const float* p) { Vec r; r.v = *reinterpret_cast<const float4*>(p); return r; }
  __device__ void store(float* p) const { *reinterpret_cast<float4*>(p) = v; }
  // bf16 deltas: 4 values = one 8-byte access, widened to / rounded from fp32 (nearest even)
  __device__ static Vec load(const mie_bf16* p) {
    const mie_bf16x4 b = *reinterpret_cast<const mie_bf16x4*>(p);
    Vec r; r.v = make_float4((float)b[0], (float)b[1], (float)b[2], (float)b[3]); return r;
  }
  __device__ void store(mie_bf16* p) const {
    mie_bf16x4 b; b[0] = (mie_bf16)v.x; b[1] = (mie_bf16)v.y; b[2] = (mie_bf16)v.z; b[3] = (mie_bf16)v.w;
    *reinterpret_cast<mie_bf16x4*>(p) = b;
  }
  __device__ static Vec zero() { Vec r; r.v = make_float4(0.f, 0.f, 0.f, 0.f); return r; }
  __device__ float& operator[](int i) { return (&v.x)[i]; }
};
// 8 channels: one 16-byte access of a bf16 delta, two of an fp32 buffer
template <> struct Vec<8> {
  float v[8];
  __device__ static Vec load(const float* p) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    Vec r; r.v[0] = a.x; r.v[1] = a.y; r.v[2] = a.z; r.v[3] = a.w; r.v[4] = b.x; r.v[5] = b.y; r.v[6] = b.z; r.v[7] = b.w;
    return r;
  }
  __device__ void store(float* p) const {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
  __device__ static Vec load(const mie_bf16* p) {
    const mie_bf16x8 b = *reinterpret_cast<const mie_bf16x8*>(p);
    Vec r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r.v[i] = (float)b[i];
    return r;
  }
  __device__ void store(mie_bf16* p) const {
    mie_bf16x8 b;
#pragma unroll
    for (int i = 0; i < 8; ++i) b[i] = (mie_bf16)v[i];
    *reinterpret_cast<mie_bf16x8*>(p) = b;
  }
  __device__ static Vec zero() { Vec r; for (int i = 0; i < 8; ++i) r.v[i] = 0.f; return r; }
  __device__ float& operator[](int i) { return v[i]; }
};
template <> struct Vec<1> {
  float v;
  __device__ static Vec load(const float* p) { Vec r; r.v = *p; return r; }
  __device__ void store(float* p) const { *p = v; }
  __device__ static Vec load(const mie_bf16* p) { Vec r; r.v = (float)*p; return r; }
  __device__ void store(mie_bf16* p) const { *p = (mie_bf16)v; }
  __device__ static Vec zero() { Vec r; r.v = 0.f; return r; }
  __device__ float& operator[](int) { return v; }
};

// Slot walker: calls f(px, pixoff, cq) for every in-bounds (pixel, channel vector) slot of
// the tile that belongs to this block; px in [0,64), pixoff = linear pixel index.  The
// channel vectors of a tile are split over gridDim.y blocks so that layers with few tiles
// (33x44: 30 tiles) still put a few hundred workgroups on the chip.
template <typename F>
__device__ __forceinline__ void for_tile_slots(const TileSetDev& ts, int n, int y0, int x0,
                                               int cv, F f) {
  const int per = (cv + (int)gridDim.y - 1) / (int)gridDim.y;
  const int cq0 = (int)blockIdx.y * per;
  const int cvb = (cv - cq0 < per) ? cv - cq0 : per;
  if (cvb <= 0) return;
  const int total = 64 * cvb;
  for (int idx = threadIdx.x; idx < total; idx += 256) {
    const int px = idx / cvb, cq = cq0 + (idx - px * cvb);
    const int y = y0 + (px >> 3), x = x0 + (px & 7);
    if (y >= ts.h || x >= ts.w) continue;
    const long long pixoff = ((long long)n * ts.h + y) * ts.w + x;
    f(px, pixoff, cq);
  }
}

// Number of channel splits (gridDim.y) for `cap` tiles and `cv` channel vectors per pixel:
// aim for >= 1024 workgroups, keep >= 4 vectors x 64 pixels = one slot per thread.
static inline unsigned channel_splits(int cap, int cv) {
  int want = (1024 + cap - 1) / cap;
  int most = cv / 4;
  if (most < 1) most = 1;
  if (want > most) want = most;
  if (want < 1) want = 1;
  return (unsigned)want;
}

// ---- activation increment -----------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(256) void k_act_incr(TileSetDev ts, int kind, float slope,
                                                  const T* din,     // may alias dout (in place)
                                                  float* __restrict__ res,
                                                  T* dout, int c,
                                                  uint8_t* __restrict__ out_mask, int keep) {
  __shared__ unsigned s_any[64];
  int n, y0, x0;
  const int tk = mie_pick_tile(ts, blockIdx.x, n, y0, x0);
  if (tk == 0) return;
  if (out_mask) {
    if (threadIdx.x < 64) s_any[threadIdx.x] = 0u;
    __syncthreads();
  }
  const int cv = c / VEC;
  for_tile_slots(ts, n, y0, x0, cv, [&](int px, long long pixoff, int cq) {
    const long long off = pixoff * c + (long long)cq * VEC;
    Vec<VEC> o = Vec<VEC>::zero();
    if (tk == 1 && ts.pixmask[pixoff]) {
      Vec<VEC> d = Vec<VEC>::load(din + off);
      Vec<VEC> r = Vec<VEC>::load(res + off);
      unsigned nz = 0u;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float r0 = r[i], r1 = r0 + d[i];
        const float v = mie_act(kind, slope, r1) - mie_act(kind, slope, r0);
        o[i] = v;
        r[i] = r1;
        nz |= (v != 0.f) ? 1u : 0u;
      }
      if (!keep) r.store(res + off);
      if (out_mask && nz) atomicOr(&s_any[px], 1u);
    }
    o.store(dout + off);
  });
  if (out_mask) {
    __syncthreads();
    if (threadIdx.x < 64) {
      const int px = threadIdx.x;
      const int y = y0 + (px >> 3), x = x0 + (px & 7);
      if (y < ts.h && x < ts.w) {
        const long long pixoff = ((long long)n * ts.h + y) * ts.w + x;
        out_mask[pixoff] = (uint8_t)((tk == 1 && s_any[px]) ? 1 : 0);
      }
    }
  }
}

// ---- delta quantiser (k-fence) ---------------------------------------------------
// t = carry + d;  f = k * floor(0.5 + t / k);  carry = t - f;  out = f.  Every operation is a
// separately rounded IEEE fp32 op (no contraction, true division), so the result equals the
// same expression evaluated op by op on the host.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void k_kfence_incr(TileSetDev ts, const float* __restrict__ k_dev,
                                                     float k_host, const T* din,   // may alias dout
                                                     float* __restrict__ carry,
                                                     T* dout, int c,
                                                     uint8_t* __restrict__ out_mask) {
  __shared__ unsigned s_any[64];
  int n, y0, x0;
  const int tk = mie_pick_tile(ts, blockIdx.x, n, y0, x0);
  if (tk == 0) return;
  if (out_mask) {
    if (threadIdx.x < 64) s_any[threadIdx.x] = 0u;
    __syncthreads();
  }
  const float k = k_dev ? *k_dev : k_host;
  const bool fence = k > 0.f && k < INFINITY;     // otherwise the delta passes unchanged
  const int cv = c / VEC;
  for_tile_slots(ts, n, y0, x0, cv, [&](int px, long long pixoff, int cq) {
    const long long off = pixoff * c + (long long)cq * VEC;
    Vec<VEC> o = Vec<VEC>::zero();
    if (tk == 1 && ts.pixmask[pixoff]) {
      Vec<VEC> d = Vec<VEC>::load(din + off);
      Vec<VEC> r = Vec<VEC>::load(carry + off);
      unsigned nz = 0u;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float t = __fadd_rn(r[i], d[i]);
        const float f = fence ? __fmul_rn(k, floorf(__fadd_rn(0.5f, __fdiv_rn(t, k)))) : t;
        o[i] = f;
        r[i] = __fsub_rn(t, f);
        nz |= (f != 0.f) ? 1u : 0u;
      }
      r.store(carry + off);
      if (out_mask && nz) atomicOr(&s_any[px], 1u);
    }
    o.store(dout + off);
  });
  if (out_mask) {
    __syncthreads();
    if (threadIdx.x < 64) {
      const int px = threadIdx.x;
      const int y = y0 + (px >> 3), x = x0 + (px & 7);
      if (y < ts.h && x < ts.w) {
        const long long pixoff = ((long long)n * ts.h + y) * ts.w + x;
        out_mask[pixoff] = (uint8_t)((tk == 1 && s_any[px]) ? 1 : 0);
      }
    }
  }
}

// ---- product rule ---------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(256) void k_mul_incr(TileSetDev ts, const T* __restrict__ d1,
                                                  const uint8_t* __restrict__ m1,
                                                  float* __restrict__ r1,
                                                  const T* __restrict__ d2,
                                                  const uint8_t* __restrict__ m2,
                                                  float* __restrict__ r2,
                                                  T* __restrict__ dout, int c, int keep) {
  int n, y0, x0;
  const int tk = mie_pick_tile(ts, blockIdx.x, n, y0, x0);
  if (tk == 0) return;
  const int cv = c / VEC;
  for_tile_slots(ts, n, y0, x0, cv, [&](int, long long pixoff, int cq) {
    const long long off = pixoff * c + (long long)cq * VEC;
    Vec<VEC> o = Vec<VEC>::zero();
    if (tk == 1 && ts.pixmask[pixoff]) {
      const bool a1 = (m1 == nullptr) || m1[pixoff];
      const bool a2 = (m2 == nullptr) || m2[pixoff];
      if (a1 || a2) {
        Vec<VEC> x1 = a1 ? Vec<VEC>::load(d1 + off) : Vec<VEC>::zero();
        Vec<VEC> x2 = a2 ? Vec<VEC>::load(d2 + off) : Vec<VEC>::zero();
        Vec<VEC> q1 = Vec<VEC>::load(r1 + off);
        Vec<VEC> q2 = Vec<VEC>::load(r2 + off);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          o[i] = (x2[i] + q2[i]) * x1[i] + q1[i] * x2[i];
          q1[i] += x1[i];
          q2[i] += x2[i];
        }
        if (a1 && !keep) q1.store(r1 + off);
        if (a2 && !keep) q2.store(r2 + off);
      }
    }
    o.store(dout + off);
  });
}

// ---- sum ----------------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(256) void k_add_incr(TileSetDev ts, const T* __restrict__ a,
                                                  const uint8_t* __restrict__ ma,
                                                  const T* __restrict__ b,
                                                  const uint8_t* __restrict__ mb,
                                                  T* __restrict__ dout, int c) {
  int n, y0, x0;
  const int tk = mie_pick_tile(ts, blockIdx.x, n, y0, x0);
  if (tk == 0) return;
  const int cv = c / VEC;
  for_tile_slots(ts, n, y0, x0, cv, [&](int, long long pixoff, int cq) {
    const long long off = pixoff * c + (long long)cq * VEC;
    Vec<VEC> o = Vec<VEC>::zero();
    if (tk == 1 && ts.pixmask[pixoff]) {
      if (ma == nullptr || ma[pixoff]) o = Vec<VEC>::load(a + off);
      if (mb == nullptr || mb[pixoff]) {
        Vec<VEC> t = Vec<VEC>::load(b + off);
#pragma unroll
        for (int i = 0; i < VEC; ++i) o[i] += t[i];
      }
    }
    o.store(dout + off);
  });
}

// ---- bilinear x2 ------------------------------------------------------------------
// Source rows/cols and weights of output index o (align_corners = False,
// scale 2): src = max(0, o/2 - 0.25).
__device__ __forceinline__ void up2x_coef(int o, int in_size, int& i0, int& i1, float& l0,
                                          float& l1) {
  const int j = o >> 1;
  if (o & 1) {
    i0 = j; i1 = (j + 1 < in_size) ? j + 1 : j; l0 = 0.75f; l1 = 0.25f;
  } else if (j == 0) {
    i0 = 0; i1 = (1 < in_size) ? 1 : 0; l0 = 1.f; l1 = 0.f;
  } else {
    i0 = j - 1; i1 = j; l0 = 0.25f; l1 = 0.75f;
  }
}

// One workgroup per 8x8 output tile (and channel range).  The tile's outputs blend a 6x6 block of source
// pixels (rows y0/2-1 .. y0/2+4): the block is summed (a + b, masked) into LDS once, fp32, and every
// output slot then reads its four taps from there -- 36 source pixels fetched per tile instead of
// 4 per output pixel, which is what the kernel was bound by (load instructions, not bytes).
template <typename T, int VEC>
__device__ __forceinline__ void up2x_tile(const TileSetDev& ts, const T* __restrict__ a,
                                          const uint8_t* __restrict__ ma, const T* __restrict__ b,
                                          const uint8_t* __restrict__ mb, int h_in, int w_in,
                                          T* __restrict__ dout, int c) {
  extern __shared__ __attribute__((aligned(16))) float s_src[];   // [36 source pixels][channels of this block]
  __shared__ uint8_t s_act[64];                                   // output pixel active (fetched with the sources)
  int n, y0, x0;
  const int tk = mie_pick_tile(ts, blockIdx.x, n, y0, x0);
  if (tk == 0) return;
  const int cv = c / VEC;
  const int per = (cv + (int)gridDim.y - 1) / (int)gridDim.y;     // the channel split of for_tile_slots
  const int cq0 = (int)blockIdx.y * per;
  const int cvb = (cv - cq0 < per) ? cv - cq0 : per;
  if (cvb <= 0) return;
  const int cw = cvb * VEC;
  const int ry0 = (y0 >> 1) - 1, rx0 = (x0 >> 1) - 1;
  if (tk == 1) {
    if (threadIdx.x < 64) {
      const int oy = y0 + ((int)threadIdx.x >> 3), ox = x0 + ((int)threadIdx.x & 7);
      s_act[threadIdx.x] = (oy < ts.h && ox < ts.w) ? ts.pixmask[((long long)n * ts.h + oy) * ts.w + ox] : 0;
    }
    for (int idx = threadIdx.x; idx < 36 * cvb; idx += 256) {
      const int sp = idx / cvb, cq = idx - sp * cvb;
      const int sy = ry0 + sp / 6, sx = rx0 + sp % 6;
      Vec<VEC> t = Vec<VEC>::zero();
      if (sy >= 0 && sy < h_in && sx >= 0 && sx < w_in) {
        const long long so = ((long long)n * h_in + sy) * w_in + sx;
        const long long eo = so * c + (long long)(cq0 + cq) * VEC;
        if (ma == nullptr || ma[so]) t = Vec<VEC>::load(a + eo);
        if (b != nullptr && (mb == nullptr || mb[so])) {
          Vec<VEC> u = Vec<VEC>::load(b + eo);
#pragma unroll
          for (int e = 0; e < VEC; ++e) t[e] += u[e];
        }
      }
      t.store(s_src + sp * cw + cq * VEC);
    }
    __syncthreads();
  }
  for_tile_slots(ts, n, y0, x0, cv, [&](int px, long long pixoff, int cq) {
    const long long off = pixoff * c + (long long)cq * VEC;
    Vec<VEC> o = Vec<VEC>::zero();
    if (tk == 1 && s_act[px]) {
      const int oy = y0 + (px >> 3), ox = x0 + (px & 7);
      int r[2], q[2];
      float lr[2], lq[2];
      up2x_coef(oy, h_in, r[0], r[1], lr[0], lr[1]);
      up2x_coef(ox, w_in, q[0], q[1], lq[0], lq[1]);
      // value(i,j) = a + b at source (r[i], q[j]); combine as torch does:
      // l_r0*(l_c0*v00 + l_c1*v01) + l_r1*(l_c0*v10 + l_c1*v11)
      Vec<VEC> v[2][2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          v[i][j] = Vec<VEC>::load(static_cast<const float*>(s_src) + ((r[i] - ry0) * 6 + (q[j] - rx0)) * cw +
                                   (cq - cq0) * VEC);
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        o[e] = lr[0] * (lq[0] * v[0][0][e] + lq[1] * v[0][1][e]) +
               lr[1] * (lq[0] * v[1][0][e] + lq[1] * v[1][1][e]);
    }
    o.store(dout + off);
  });
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void k_up2x_incr(TileSetDev ts, const T* __restrict__ a,
                                                   const uint8_t* __restrict__ ma,
                                                   const T* __restrict__ b,
                                                   const uint8_t* __restrict__ mb, int h_in,
                                                   int w_in, T* __restrict__ dout, int c) {
  up2x_tile<T, VEC>(ts, a, ma, b, mb, h_in, w_in, dout, c);
}

// Two independent up-samplings of the same geometry (tensors, masks and tile sets of their own) in one
// launch: blockIdx.z picks the operand set.  For decoders that up-sample the parts of a concat one by one.
template <typename T>
struct Up2xSet {
  TileSetDev ts; const T* a; const uint8_t* ma; T* out;
};
template <typename T, int VEC>
__global__ __launch_bounds__(256) void k_up2x_pair(Up2xSet<T> s0, Up2xSet<T> s1, int h_in, int w_in, int c) {
  if (blockIdx.z == 0) up2x_tile<T, VEC>(s0.ts, s0.a, s0.ma, (const T*)nullptr, (const uint8_t*)nullptr, h_in, w_in, s0.out, c);
  else up2x_tile<T, VEC>(s1.ts, s1.a, s1.ma, (const T*)nullptr, (const uint8_t*)nullptr, h_in, w_in, s1.out, c);
}

// ---- max pooling increment and masked accumulate ---------------------------------
// out = pool(R + d) - pool(R) over the active output tiles (window taps outside the image are
// skipped, which is the -inf padding of torch's max_pool2d); R itself is only read here, the
// caller accumulates it afterwards with k_accumulate (windows of neighbouring tiles overlap, so
// an in-place update inside this kernel would race).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void k_maxpool_incr(TileSetDev ts, const T* __restrict__ din,
                                                      const uint8_t* __restrict__ dmask,
                                                      const float* __restrict__ res, int h_in, int w_in,
                                                      int c, int k, int s, int pad, T* __restrict__ dout) {
  int n, y0, x0;
  const int tk = mie_pick_tile(ts, blockIdx.x, n, y0, x0);
  if (tk == 0) return;
  const int cv = c / VEC;
  for_tile_slots(ts, n, y0, x0, cv, [&](int px, long long pixoff, int cq) {
    const long long off = pixoff * c + (long long)cq * VEC;
    Vec<VEC> o = Vec<VEC>::zero();
    if (tk == 1 && ts.pixmask[pixoff]) {
      const int oy = y0 + (px >> 3), ox = x0 + (px & 7);
      Vec<VEC> m0, m1;
#pragma unroll
      for (int e = 0; e < VEC; ++e) m0[e] = m1[e] = -INFINITY;
      for (int ky = 0; ky < k; ++ky) {
        const int iy = oy * s - pad + ky;
        if (iy < 0 || iy >= h_in) continue;
        for (int kx = 0; kx < k; ++kx) {
          const int ix = ox * s - pad + kx;
          if (ix < 0 || ix >= w_in) continue;
          const long long so = ((long long)n * h_in + iy) * w_in + ix;
          Vec<VEC> r = Vec<VEC>::load(res + so * c + (long long)cq * VEC);
          Vec<VEC> d = (dmask == nullptr || dmask[so]) ? Vec<VEC>::load(din + so * c + (long long)cq * VEC)
                                                       : Vec<VEC>::zero();
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            m0[e] = fmaxf(m0[e], r[e]);
            m1[e] = fmaxf(m1[e], r[e] + d[e]);
          }
        }
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) o[e] = m1[e] - m0[e];
    }
    o.store(dout + off);
  });
}

// R += d at the active pixels of the tile set (IncrementReserve.accumulate without touching the
// rest of the frame).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void k_accumulate(TileSetDev ts, const T* __restrict__ din,
                                                    float* __restrict__ res, int c) {
  int n, y0, x0;
  const int tk = mie_pick_tile(ts, blockIdx.x, n, y0, x0);
  if (tk != 1) return;
  const int cv = c / VEC;
  for_tile_slots(ts, n, y0, x0, cv, [&](int, long long pixoff, int cq) {
    if (!ts.pixmask[pixoff]) return;
    const long long off = pixoff * c + (long long)cq * VEC;
    Vec<VEC> r = Vec<VEC>::load(res + off);
    Vec<VEC> d = Vec<VEC>::load(din + off);
#pragma unroll
    for (int e = 0; e < VEC; ++e) r[e] += d[e];
    r.store(res + off);
  });
}

// ---- fused ConvLSTM gates ------------------------------------------------------

template <typename T, int VEC>
__global__ __launch_bounds__(256) void k_convlstm_gates(
    TileSetDev ts, const T* __restrict__ dg, float* __restrict__ gres,
    const T* __restrict__ dcp, const uint8_t* __restrict__ mcp, float* __restrict__ cpres,
    float* __restrict__ cres, T* __restrict__ dh, T* __restrict__ dc, int hid) {
  int n, y0, x0;
  const int tk = mie_pick_tile(ts, blockIdx.x, n, y0, x0);
  if (tk == 0) return;
  const int cv = hid / VEC;
  for_tile_slots(ts, n, y0, x0, cv, [&](int, long long pixoff, int cq) {
    const long long off = pixoff * hid + (long long)cq * VEC;
    Vec<VEC> oh = Vec<VEC>::zero(), oc = Vec<VEC>::zero();
    if (tk == 1 && ts.pixmask[pixoff]) {
      const long long goff = pixoff * 4 * hid + (long long)cq * VEC;
      Vec<VEC> di = Vec<VEC>::load(dg + goff), ri = Vec<VEC>::load(gres + goff);
      Vec<VEC> df = Vec<VEC>::load(dg + goff + hid), rf = Vec<VEC>::load(gres + goff + hid);
      Vec<VEC> dO = Vec<VEC>::load(dg + goff + 2 * hid), ro = Vec<VEC>::load(gres + goff + 2 * hid);
      Vec<VEC> dG = Vec<VEC>::load(dg + goff + 3 * hid), rg = Vec<VEC>::load(gres + goff + 3 * hid);
      const bool has_cp = (dcp != nullptr) && (mcp == nullptr || mcp[pixoff]);
      Vec<VEC> dP = has_cp ? Vec<VEC>::load(dcp + off) : Vec<VEC>::zero();
      Vec<VEC> cp = Vec<VEC>::load(cpres + off);
      Vec<VEC> cc = Vec<VEC>::load(cres + off);
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        mie_lstm_gate_chain(ri[e], rf[e], ro[e], rg[e], di[e], df[e], dO[e], dG[e], cp[e], dP[e], cc[e], oh[e],
                            oc[e]);
      ri.store(gres + goff); rf.store(gres + goff + hid);
      ro.store(gres + goff + 2 * hid); rg.store(gres + goff + 3 * hid);
      if (has_cp) cp.store(cpres + off);
      cc.store(cres + off);
    }
    oh.store(dh + off);
    oc.store(dc + off);
  });
}

// ---- fused ConvGRU gates (state reset each step: new_state = candidate * update) ---------------

// dg is [n,h,w,2*hid]: the update-gate conv delta in channels [0, hid), the candidate conv delta in [hid, 2*hid).
// Per element: du, dc -> d(sigmoid), d(tanh) on the pre-activation reservoirs, then the product rule with the
// cached operands recomputed from those reservoirs: dh = (ds + s0) * dt + t0 * ds.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void k_convgru_gates(TileSetDev ts, const T* __restrict__ dg,
                                                       float* __restrict__ ures, float* __restrict__ cres,
                                                       T* __restrict__ dh, int hid) {
  int n, y0, x0;
  const int tk = mie_pick_tile(ts, blockIdx.x, n, y0, x0);
  if (tk == 0) return;
  const int cv = hid / VEC;
  for_tile_slots(ts, n, y0, x0, cv, [&](int, long long pixoff, int cq) {
    const long long off = pixoff * hid + (long long)cq * VEC;
    Vec<VEC> oh = Vec<VEC>::zero();
    if (tk == 1 && ts.pixmask[pixoff]) {
      const long long goff = pixoff * 2 * hid + (long long)cq * VEC;
      Vec<VEC> du = Vec<VEC>::load(dg + goff), ru = Vec<VEC>::load(ures + off);
      Vec<VEC> dc = Vec<VEC>::load(dg + goff + hid), rc = Vec<VEC>::load(cres + off);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float ru1 = ru[e] + du[e], rc1 = rc[e] + dc[e];
        const float s0 = mie_sigm(ru[e]), ds = mie_sigm(ru1) - s0;
        const float t0 = tanhf(rc[e]), dt = tanhf(rc1) - t0;
        oh[e] = (ds + s0) * dt + t0 * ds;             // IncrPointwiseMultiply(candidate, update)
        ru[e] = ru1;
        rc[e] = rc1;
      }
      ru.store(ures + off);
      rc.store(cres + off);
    }
    oh.store(dh + off);
  });
}

int check_pointwise(const char* who, const mie_tileset* ts, int c) {
  int rc = mie_check_tileset(ts, who);
  if (rc != MIE_OK) return rc;
  MIE_REQUIRE(c > 0 && c <= 65536, MIE_ERR_INVALID_ARG, "%s: channel count %d out of range", who, c);
  return MIE_OK;
}

#define MIE_PTR16(p, who, name) \
  MIE_REQUIRE(mie_aligned((p), 16), MIE_ERR_INVALID_ARG, "%s: %s must be 16-byte aligned", who, name)

// Launches KERN<T, VEC> with T from `dtype` and VEC = 4 when c % 4 == 0, else 1.  The kernel
// arguments are built by ARGS, a macro-local expression list that may use T.
// Launches KERN<T, VEC> with T from `dtype`; VEC = 8 for bf16 deltas with c % 8 == 0 (16-byte
// delta accesses), else 4 when c % 4 == 0, else 1.  SPLIT: whether the channel vectors of a tile
// may be spread over gridDim.y.  The kernel arguments may use T.
#define MIE_LAUNCH_VEC(KERN, T_, VEC_, c, grid, SPLIT, stream, ...)                                        \
  do {                                                                                                    \
    using T = T_;                                                                                         \
    const unsigned ny_ = (SPLIT) ? channel_splits((int)(grid), (c) / (VEC_)) : 1u;                        \
    hipLaunchKernelGGL((KERN<T, VEC_>), dim3(grid, ny_), dim3(256), 0, (hipStream_t)(stream), __VA_ARGS__); \
  } while (0)

#define MIE_LAUNCH_POINTWISE(KERN, dtype, c, grid, SPLIT, stream, ...)                                     \
  do {                                                                                                    \
    if ((dtype) == MIE_DTYPE_BF16) {                                                                      \
      if (((c) & 7) == 0) MIE_LAUNCH_VEC(KERN, mie_bf16, 8, c, grid, SPLIT, stream, __VA_ARGS__);         \
      else if (((c) & 3) == 0) MIE_LAUNCH_VEC(KERN, mie_bf16, 4, c, grid, SPLIT, stream, __VA_ARGS__);    \
      else MIE_LAUNCH_VEC(KERN, mie_bf16, 1, c, grid, SPLIT, stream, __VA_ARGS__);                        \
    } else {                                                                                              \
      if (((c) & 7) == 0 && (c) >= 64) MIE_LAUNCH_VEC(KERN, float, 8, c, grid, SPLIT, stream, __VA_ARGS__); \
      else if (((c) & 3) == 0) MIE_LAUNCH_VEC(KERN, float, 4, c, grid, SPLIT, stream, __VA_ARGS__);       \
      else MIE_LAUNCH_VEC(KERN, float, 1, c, grid, SPLIT, stream, __VA_ARGS__);                           \
    }                                                                                                     \
  } while (0)

#define MIE_DTYPE_OK(dtype, who)                                                                      \
  MIE_REQUIRE((dtype) == MIE_DTYPE_F32 || (dtype) == MIE_DTYPE_BF16, MIE_ERR_UNSUPPORTED,              \
              "%s: unknown delta dtype %d", who, (int)(dtype))

}  // namespace

extern "C" int mie_act_incr(int act_kind, float slope, const void* in_delta, float* reservoir,
                            void* out_delta, int c, const mie_tileset* ts,
                            uint8_t* out_pixmask, int flags, int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_act_incr";
  int rc = check_pointwise(who, ts, c);
  if (rc != MIE_OK) return rc;
  MIE_DTYPE_OK(dtype, who);
  MIE_REQUIRE(in_delta && reservoir && out_delta, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(act_kind >= MIE_ACT_NONE && act_kind <= MIE_ACT_TANH, MIE_ERR_UNSUPPORTED,
              "%s: unknown activation %d", who, act_kind);
  MIE_PTR16(in_delta, who, "in_delta"); MIE_PTR16(reservoir, who, "reservoir");
  MIE_PTR16(out_delta, who, "out_delta");
  const int keep = (flags & MIE_FLAG_KEEP_RESERVOIR) ? 1 : 0;
  const TileSetDev d = mie_dev_tileset(ts);
  const unsigned grid = (unsigned)mie_tile_capacity(ts->n, ts->h, ts->w);
  // the refined mask is an any-over-channels inside one block: no channel split then
  MIE_LAUNCH_POINTWISE(k_act_incr, dtype, c, grid, out_pixmask == nullptr, stream, d, act_kind, slope, (const T*)in_delta,
                       reservoir, (T*)out_delta, c, out_pixmask, keep);
  return mie_check_launch(who);
}

extern "C" int mie_kfence_incr(const void* in_delta, float* carry, const float* k_dev, float k_host,
                               void* out_delta, int c, const mie_tileset* ts,
                               uint8_t* out_pixmask, int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_kfence_incr";
  int rc = check_pointwise(who, ts, c);
  if (rc != MIE_OK) return rc;
  MIE_DTYPE_OK(dtype, who);
  MIE_REQUIRE(in_delta && carry && out_delta, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE((const void*)carry != in_delta && (void*)carry != out_delta, MIE_ERR_INVALID_ARG,
              "%s: the carry must not alias a delta", who);
  MIE_REQUIRE(k_dev != nullptr || (k_host > 0.f && k_host < INFINITY), MIE_ERR_INVALID_ARG,
              "%s: k = %g must be positive and finite", who, (double)k_host);
  MIE_PTR16(in_delta, who, "in_delta"); MIE_PTR16(carry, who, "carry");
  MIE_PTR16(out_delta, who, "out_delta");
  MIE_REQUIRE(mie_aligned(k_dev, 4), MIE_ERR_INVALID_ARG, "%s: k_dev must be 4-byte aligned", who);
  const TileSetDev d = mie_dev_tileset(ts);
  const unsigned grid = (unsigned)mie_tile_capacity(ts->n, ts->h, ts->w);
  MIE_LAUNCH_POINTWISE(k_kfence_incr, dtype, c, grid, out_pixmask == nullptr, stream, d, k_dev, k_host, (const T*)in_delta,
                       carry, (T*)out_delta, c, out_pixmask);
  return mie_check_launch(who);
}

extern "C" int mie_mul_incr(const void* d1, const uint8_t* m1, float* r1, const void* d2,
                            const uint8_t* m2, float* r2, void* out_delta, int c,
                            const mie_tileset* ts, int flags, int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_mul_incr";
  int rc = check_pointwise(who, ts, c);
  if (rc != MIE_OK) return rc;
  MIE_DTYPE_OK(dtype, who);
  MIE_REQUIRE(d1 && r1 && d2 && r2 && out_delta, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_PTR16(d1, who, "d1"); MIE_PTR16(r1, who, "r1"); MIE_PTR16(d2, who, "d2");
  MIE_PTR16(r2, who, "r2"); MIE_PTR16(out_delta, who, "out_delta");
  const int keep = (flags & MIE_FLAG_KEEP_RESERVOIR) ? 1 : 0;
  const TileSetDev d = mie_dev_tileset(ts);
  const unsigned grid = (unsigned)mie_tile_capacity(ts->n, ts->h, ts->w);
  MIE_LAUNCH_POINTWISE(k_mul_incr, dtype, c, grid, true, stream, d, (const T*)d1, m1, r1, (const T*)d2, m2, r2,
                       (T*)out_delta, c, keep);
  return mie_check_launch(who);
}

extern "C" int mie_add_incr(const void* a, const uint8_t* ma, const void* b, const uint8_t* mb,
                            void* out_delta, int c, const mie_tileset* ts, int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_add_incr";
  int rc = check_pointwise(who, ts, c);
  if (rc != MIE_OK) return rc;
  MIE_DTYPE_OK(dtype, who);
  MIE_REQUIRE(a && b && out_delta, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_PTR16(a, who, "a"); MIE_PTR16(b, who, "b"); MIE_PTR16(out_delta, who, "out_delta");
  const TileSetDev d = mie_dev_tileset(ts);
  const unsigned grid = (unsigned)mie_tile_capacity(ts->n, ts->h, ts->w);
  MIE_LAUNCH_POINTWISE(k_add_incr, dtype, c, grid, true, stream, d, (const T*)a, ma, (const T*)b, mb,
                       (T*)out_delta, c);
  return mie_check_launch(who);
}

extern "C" int mie_upsample2x_incr(const void* a, const uint8_t* ma, const void* b,
                                   const uint8_t* mb, int h_in, int w_in, int c,
                                   const mie_tileset* out, void* out_delta, int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_upsample2x_incr";
  int rc = check_pointwise(who, out, c);
  if (rc != MIE_OK) return rc;
  MIE_DTYPE_OK(dtype, who);
  MIE_REQUIRE(a && out_delta, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(b != nullptr || mb == nullptr, MIE_ERR_INVALID_ARG, "%s: mask of absent input b", who);
  MIE_REQUIRE(h_in > 0 && w_in > 0 && out->h == 2 * h_in && out->w == 2 * w_in,
              MIE_ERR_INVALID_ARG, "%s: output (%d,%d) is not twice the input (%d,%d)", who,
              out->h, out->w, h_in, w_in);
  MIE_PTR16(a, who, "a"); MIE_PTR16(b, who, "b"); MIE_PTR16(out_delta, who, "out_delta");
  const TileSetDev d = mie_dev_tileset(out);
  const unsigned grid = (unsigned)mie_tile_capacity(out->n, out->h, out->w);
  // channel vectors per block bounded so that the 36-pixel source block fits 36 KB of LDS
  const bool bf = dtype == MIE_DTYPE_BF16;
  const int vec = (c % 8 == 0 && (bf || c >= 64)) ? 8 : (c % 4 == 0 ? 4 : 1);
  const int cv = c / vec;
  unsigned ny = channel_splits((int)grid, cv);
  const unsigned ny_min = (unsigned)mie_div_up(c, 256);
  if (ny < ny_min) ny = ny_min;
  const size_t lds = (size_t)36 * mie_div_up(cv, (int)ny) * vec * sizeof(float);
#define MIE_UP2X_LAUNCH(T_, V_)                                                                              \
  hipLaunchKernelGGL((k_up2x_incr<T_, V_>), dim3(grid, ny), dim3(256), lds, (hipStream_t)stream, d, (const T_*)a, \
                     ma, (const T_*)b, mb, h_in, w_in, (T_*)out_delta, c)
  if (bf) {
    if (vec == 8) MIE_UP2X_LAUNCH(mie_bf16, 8); else if (vec == 4) MIE_UP2X_LAUNCH(mie_bf16, 4); else MIE_UP2X_LAUNCH(mie_bf16, 1);
  } else {
    if (vec == 8) MIE_UP2X_LAUNCH(float, 8); else if (vec == 4) MIE_UP2X_LAUNCH(float, 4); else MIE_UP2X_LAUNCH(float, 1);
  }
#undef MIE_UP2X_LAUNCH
  return mie_check_launch(who);
}

extern "C" int mie_upsample2x_pair_incr(const void* a0, const uint8_t* m0, const mie_tileset* out0, void* out_delta0,
                                        const void* a1, const uint8_t* m1, const mie_tileset* out1, void* out_delta1,
                                        int h_in, int w_in, int c, int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_upsample2x_pair_incr";
  int rc = check_pointwise(who, out0, c);
  if (rc != MIE_OK) return rc;
  rc = check_pointwise(who, out1, c);
  if (rc != MIE_OK) return rc;
  MIE_DTYPE_OK(dtype, who);
  MIE_REQUIRE(a0 && a1 && out_delta0 && out_delta1, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(out_delta0 != out_delta1 && out0 != out1 && out0->tiles != out1->tiles, MIE_ERR_INVALID_ARG,
              "%s: the two outputs and tile sets must be distinct", who);
  MIE_REQUIRE(h_in > 0 && w_in > 0 && out0->h == 2 * h_in && out0->w == 2 * w_in && out1->h == out0->h &&
                  out1->w == out0->w && out1->n == out0->n,
              MIE_ERR_INVALID_ARG, "%s: both outputs must be (n, %d, %d), twice the input", who, 2 * h_in, 2 * w_in);
  MIE_PTR16(a0, who, "a0"); MIE_PTR16(a1, who, "a1"); MIE_PTR16(out_delta0, who, "out_delta0");
  MIE_PTR16(out_delta1, who, "out_delta1");
  const unsigned grid = (unsigned)mie_tile_capacity(out0->n, out0->h, out0->w);
  const bool bf = dtype == MIE_DTYPE_BF16;
  const int vec = (c % 8 == 0 && (bf || c >= 64)) ? 8 : (c % 4 == 0 ? 4 : 1);
  const int cv = c / vec;
  unsigned ny = channel_splits((int)grid, cv);
  const unsigned ny_min = (unsigned)mie_div_up(c, 256);
  if (ny < ny_min) ny = ny_min;
  const size_t lds = (size_t)36 * mie_div_up(cv, (int)ny) * vec * sizeof(float);
#define MIE_UP2X_PAIR(T_, V_)                                                                                  \
  do {                                                                                                         \
    Up2xSet<T_> s0{mie_dev_tileset(out0), (const T_*)a0, m0, (T_*)out_delta0};                                  \
    Up2xSet<T_> s1{mie_dev_tileset(out1), (const T_*)a1, m1, (T_*)out_delta1};                                  \
    hipLaunchKernelGGL((k_up2x_pair<T_, V_>), dim3(grid, ny, 2), dim3(256), lds, (hipStream_t)stream, s0, s1,  \
                       h_in, w_in, c);                                                                         \
  } while (0)
  if (bf) {
    if (vec == 8) MIE_UP2X_PAIR(mie_bf16, 8); else if (vec == 4) MIE_UP2X_PAIR(mie_bf16, 4); else MIE_UP2X_PAIR(mie_bf16, 1);
  } else {
    if (vec == 8) MIE_UP2X_PAIR(float, 8); else if (vec == 4) MIE_UP2X_PAIR(float, 4); else MIE_UP2X_PAIR(float, 1);
  }
#undef MIE_UP2X_PAIR
  return mie_check_launch(who);
}

extern "C" int mie_convlstm_gates_incr(const void* gates_delta, float* gates_res,
                                       const void* cprev_delta, const uint8_t* cprev_mask,
                                       float* cprev_res, float* cell_res, void* h_delta,
                                       void* c_delta, int hid, const mie_tileset* ts, int dtype,
                                       void* stream) {
  mie_clear_error();
  const char* who = "mie_convlstm_gates_incr";
  int rc = check_pointwise(who, ts, hid);
  if (rc != MIE_OK) return rc;
  MIE_DTYPE_OK(dtype, who);
  MIE_REQUIRE(gates_delta && gates_res && cprev_res && cell_res && h_delta && c_delta,
              MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(cprev_delta != nullptr || cprev_mask == nullptr, MIE_ERR_INVALID_ARG,
              "%s: mask of absent cprev_delta", who);
  MIE_PTR16(gates_delta, who, "gates_delta"); MIE_PTR16(gates_res, who, "gates_res");
  MIE_PTR16(cprev_delta, who, "cprev_delta"); MIE_PTR16(cprev_res, who, "cprev_res");
  MIE_PTR16(cell_res, who, "cell_res"); MIE_PTR16(h_delta, who, "h_delta");
  MIE_PTR16(c_delta, who, "c_delta");
  const TileSetDev d = mie_dev_tileset(ts);
  const unsigned grid = (unsigned)mie_tile_capacity(ts->n, ts->h, ts->w);
  MIE_LAUNCH_POINTWISE(k_convlstm_gates, dtype, hid, grid, true, stream, d, (const T*)gates_delta, gates_res,
                       (const T*)cprev_delta, cprev_mask, cprev_res, cell_res, (T*)h_delta, (T*)c_delta, hid);
  return mie_check_launch(who);
}

extern "C" int mie_convgru_gates_incr(const void* gates_delta, float* update_res, float* cand_res,
                                      void* h_delta, int hid, const mie_tileset* ts, int dtype,
                                      void* stream) {
  mie_clear_error();
  const char* who = "mie_convgru_gates_incr";
  int rc = check_pointwise(who, ts, hid);
  if (rc != MIE_OK) return rc;
  MIE_DTYPE_OK(dtype, who);
  MIE_REQUIRE(gates_delta && update_res && cand_res && h_delta, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(update_res != cand_res && gates_delta != h_delta, MIE_ERR_INVALID_ARG,
              "%s: the two reservoirs, and gates_delta and h_delta, must be distinct", who);
  MIE_PTR16(gates_delta, who, "gates_delta"); MIE_PTR16(update_res, who, "update_res");
  MIE_PTR16(cand_res, who, "cand_res"); MIE_PTR16(h_delta, who, "h_delta");
  const TileSetDev d = mie_dev_tileset(ts);
  const unsigned grid = (unsigned)mie_tile_capacity(ts->n, ts->h, ts->w);
  MIE_LAUNCH_POINTWISE(k_convgru_gates, dtype, hid, grid, true, stream, d, (const T*)gates_delta, update_res,
                       cand_res, (T*)h_delta, hid);
  return mie_check_launch(who);
}

extern "C" int mie_maxpool_incr(const void* in_delta, const uint8_t* in_mask, const float* reservoir,
                                int h_in, int w_in, int c, int k, int stride, int pad,
                                const mie_tileset* out, void* out_delta, int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_maxpool_incr";
  int rc = check_pointwise(who, out, c);
  if (rc != MIE_OK) return rc;
  MIE_DTYPE_OK(dtype, who);
  MIE_REQUIRE(in_delta && reservoir && out_delta, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(in_delta != out_delta, MIE_ERR_INVALID_ARG, "%s: out_delta must not alias in_delta", who);
  MIE_REQUIRE(h_in > 0 && w_in > 0 && k >= 1 && k <= 15 && stride >= 1 && stride <= 8 && pad >= 0 &&
                  2 * pad <= k,
              MIE_ERR_UNSUPPORTED, "%s: k=%d stride=%d pad=%d not implemented", who, k, stride, pad);
  MIE_REQUIRE(h_in + 2 * pad >= k && w_in + 2 * pad >= k && out->h == (h_in + 2 * pad - k) / stride + 1 &&
                  out->w == (w_in + 2 * pad - k) / stride + 1,
              MIE_ERR_INVALID_ARG, "%s: pooling (%d,%d) with k=%d s=%d p=%d does not give the tile set's (%d,%d)",
              who, h_in, w_in, k, stride, pad, out->h, out->w);
  MIE_PTR16(in_delta, who, "in_delta"); MIE_PTR16(reservoir, who, "reservoir");
  MIE_PTR16(out_delta, who, "out_delta");
  const TileSetDev d = mie_dev_tileset(out);
  const unsigned grid = (unsigned)mie_tile_capacity(out->n, out->h, out->w);
  MIE_LAUNCH_POINTWISE(k_maxpool_incr, dtype, c, grid, true, stream, d, (const T*)in_delta, in_mask, reservoir,
                       h_in, w_in, c, k, stride, pad, (T*)out_delta);
  return mie_check_launch(who);
}

extern "C" int mie_accumulate(const void* in_delta, float* reservoir, int c, const mie_tileset* ts,
                              int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_accumulate";
  int rc = check_pointwise(who, ts, c);
  if (rc != MIE_OK) return rc;
  MIE_DTYPE_OK(dtype, who);
  MIE_REQUIRE(in_delta && reservoir, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_PTR16(in_delta, who, "in_delta"); MIE_PTR16(reservoir, who, "reservoir");
  const TileSetDev d = mie_dev_tileset(ts);
  const unsigned grid = (unsigned)mie_tile_capacity(ts->n, ts->h, ts->w);
  MIE_LAUNCH_POINTWISE(k_accumulate, dtype, c, grid, true, stream, d, (const T*)in_delta, reservoir, c);
  return mie_check_launch(who);
}
