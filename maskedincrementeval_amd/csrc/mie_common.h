// Shared host/device helpers of libmie_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

// The C ABI is the only thing exported from the library.
#pragma GCC visibility push(default)
#include "../../include/mie.h"
#pragma GCC visibility pop

#define MIE_WAVE 64

// bf16 deltas (MIE_DTYPE_BF16): the compiler's native type; conversions from fp32 round to
// nearest even (v_cvt_pk_bf16_f32 on gfx950), conversions to fp32 are exact.
typedef __bf16 mie_bf16;
typedef __bf16 mie_bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 mie_bf16x8 __attribute__((ext_vector_type(8)));

// Scalar load / store of a delta element as fp32.
static __device__ __forceinline__ float mie_ld(const float* p, long long i) { return p[i]; }
static __device__ __forceinline__ float mie_ld(const mie_bf16* p, long long i) { return (float)p[i]; }
static __device__ __forceinline__ void mie_st(float* p, long long i, float v) { p[i] = v; }
static __device__ __forceinline__ void mie_st(mie_bf16* p, long long i, float v) { p[i] = (mie_bf16)v; }
// Four adjacent elements at once (i a multiple of 4, p + i 16-byte / 8-byte aligned).
static __device__ __forceinline__ float4 mie_ld4(const float* p, long long i) { return *reinterpret_cast<const float4*>(p + i); }
static __device__ __forceinline__ float4 mie_ld4(const mie_bf16* p, long long i) {
  const mie_bf16x4 b = *reinterpret_cast<const mie_bf16x4*>(p + i);
  return make_float4((float)b[0], (float)b[1], (float)b[2], (float)b[3]);
}
static __device__ __forceinline__ void mie_st4(float* p, long long i, const float4& v) { *reinterpret_cast<float4*>(p + i) = v; }
static __device__ __forceinline__ void mie_st4(mie_bf16* p, long long i, const float4& v) {
  mie_bf16x4 b;
  b[0] = (mie_bf16)v.x; b[1] = (mie_bf16)v.y; b[2] = (mie_bf16)v.z; b[3] = (mie_bf16)v.w;
  *reinterpret_cast<mie_bf16x4*>(p + i) = b;
}

// ---- host side: error reporting -------------------------------------------
void mie_set_error(const char* fmt, ...);
void mie_clear_error();

#define MIE_REQUIRE(cond, code, ...)        \
  do {                                      \
    if (!(cond)) {                          \
      mie_set_error(__VA_ARGS__);           \
      return (code);                        \
    }                                       \
  } while (0)

// Status of the launch that was just enqueued.
static inline int mie_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    mie_set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return MIE_ERR_LAUNCH;
  }
  return MIE_OK;
}

static inline bool mie_aligned(const void* p, size_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

// Validates the pointers and geometry of a tile set (host side only).
int mie_check_tileset(const mie_tileset* ts, const char* who);

static inline int mie_div_up(int a, int b) { return (a + b - 1) / b; }

// ---- device side ------------------------------------------------------------
// Plain-old-data view of a tile set passed to kernels by value.
struct TileSetDev {
  int n, h, w;
  int tiles_y, tiles_x;
  const uint8_t* pixmask;
  const int32_t* tiles;
  const int32_t* stale;
  const int32_t* counts;
};

static inline TileSetDev mie_dev_tileset(const mie_tileset* ts) {
  TileSetDev d;
  d.n = ts->n; d.h = ts->h; d.w = ts->w;
  d.tiles_y = mie_div_up(ts->h, MIE_TILE);
  d.tiles_x = mie_div_up(ts->w, MIE_TILE);
  d.pixmask = ts->pixmask; d.tiles = ts->tiles; d.stale = ts->stale;
  d.counts = ts->counts;
  return d;
}

// Which tile block `b` of a capacity-sized grid works on.
//   returns 0: nothing to do (b beyond active + stale)
//           1: active tile   2: stale tile (zero its delta)
// (n, y0, x0) = batch index and top-left output pixel of the tile.
// The same with the counts and the list entry tiles[b] already loaded by the caller (`spec`; any value
// if b is not an active position).
__device__ __forceinline__ int mie_pick_tile_loaded(const TileSetDev& ts, int b, int spec, int n_active,
                                                    int n_stale, int& n, int& y0, int& x0) {
  const int cap = ts.n * ts.tiles_y * ts.tiles_x;
  if (n_active < 0 || n_stale < 0 || n_active > cap || n_stale > cap) return 0;   // corrupt counts
  int tile, kind;
  if (b < 0) {
    return 0;
  } else if (b < n_active) {
    tile = spec;
    kind = 1;
  } else if (b < n_active + n_stale) {
    tile = ts.stale[b - n_active];
    kind = 2;
  } else {
    return 0;
  }
  if (tile < 0 || tile >= cap) return 0;    // corrupt list entry: skip rather than touch memory
  const int tx = tile % ts.tiles_x;
  const int t2 = tile / ts.tiles_x;
  const int ty = t2 % ts.tiles_y;
  n = t2 / ts.tiles_y;
  y0 = ty * MIE_TILE;
  x0 = tx * MIE_TILE;
  return kind;
}

__device__ __forceinline__ int mie_pick_tile(const TileSetDev& ts, int b,
                                             int& n, int& y0, int& x0) {
  const int cap = ts.n * ts.tiles_y * ts.tiles_x;
  // the list entry is fetched together with the counts (one memory round trip instead of two);
  // whether it is valid is decided afterwards
  const int spec = ts.tiles[(b >= 0 && b < cap) ? b : 0];
  const int n_active = ts.counts[MIE_CNT_ACTIVE];
  const int n_stale = ts.counts[MIE_CNT_STALE];
  return mie_pick_tile_loaded(ts, b, spec, n_active, n_stale, n, y0, x0);
}

__device__ __forceinline__ float mie_act(int kind, float slope, float v) {
  switch (kind) {
    case MIE_ACT_RELU: return v > 0.f ? v : 0.f;
    // __fmul_rn: keep the product from being contracted into the caller's
    // subtraction, so act(r1) - act(r0) rounds like two separate IEEE ops
    case MIE_ACT_LEAKY_RELU: return v > 0.f ? v : __fmul_rn(v, slope);
    case MIE_ACT_SIGMOID: return 1.f / (1.f + expf(-v));
    case MIE_ACT_TANH: return tanhf(v);
    default: return v;
  }
}
