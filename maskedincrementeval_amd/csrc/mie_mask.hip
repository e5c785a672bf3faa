// Pixel masks and ordered active-tile compaction (gfx950).
//
// mie_build_mask_tiles is two launches on the caller's stream: every wave of
// the first derives the 64 output-mask bits of one 8x8 tile from the input
// mask footprint and records whether the tile holds any active pixel (wave
// ballot); the second turns the per-tile flags into the ascending tile lists
// with a two-level ballot + popcount prefix scan (one block per 4096 tiles,
// each counting the flags below its chunk itself), so the list order is
// deterministic and nothing is communicated between workgroups inside a
// kernel (device-wide fences cost tens of microseconds on this chip).
#include "mie_common.h"

#include <string.h>

// ---- error string -----------------------------------------------------------
static thread_local char g_err[512] = "";

void mie_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
void mie_clear_error() { g_err[0] = 0; }

extern "C" const char* mie_last_error_string(void) { return g_err; }
extern "C" int mie_version(void) { return 100; }

extern "C" int mie_tile_capacity(int n, int h, int w) {
  if (n <= 0 || h <= 0 || w <= 0) return 0;
  long long cap = (long long)n * mie_div_up(h, MIE_TILE) * mie_div_up(w, MIE_TILE);
  if (cap > 0x3fffffff) return 0;
  return (int)cap;
}

int mie_check_tileset(const mie_tileset* ts, const char* who) {
  MIE_REQUIRE(ts != nullptr, MIE_ERR_INVALID_ARG, "%s: tile set is NULL", who);
  MIE_REQUIRE(ts->n > 0 && ts->h > 0 && ts->w > 0, MIE_ERR_INVALID_ARG,
              "%s: tile set geometry (%d,%d,%d) must be positive", who, ts->n, ts->h, ts->w);
  MIE_REQUIRE(mie_tile_capacity(ts->n, ts->h, ts->w) > 0, MIE_ERR_CAPACITY,
              "%s: tile set geometry (%d,%d,%d) too large", who, ts->n, ts->h, ts->w);
  MIE_REQUIRE((long long)ts->n * ts->h * ts->w < 0x7fffffffLL, MIE_ERR_CAPACITY,
              "%s: more than 2^31 pixels", who);
  MIE_REQUIRE(ts->pixmask && ts->tiles && ts->stale && ts->counts && ts->flags,
              MIE_ERR_INVALID_ARG, "%s: tile set has a NULL buffer", who);
  MIE_REQUIRE(mie_aligned(ts->tiles, 4) && mie_aligned(ts->stale, 4) &&
                  mie_aligned(ts->counts, 4) && mie_aligned(ts->flags, 16),
              MIE_ERR_INVALID_ARG, "%s: tile set buffers must be 4-byte aligned (flags: 16-byte)", who);
  return MIE_OK;
}

// ---- mask from delta ----------------------------------------------------------
// One thread per pixel walks its channel vector; C is small (<= 1024) and the
// vector is contiguous, float4 when the row is 16-byte aligned.
template <typename T>
__global__ __launch_bounds__(256) void k_mask_from_delta(
    const T* __restrict__ delta, long long npix, int c, float thr,
    uint8_t* __restrict__ pixmask) {
  const long long p = (long long)blockIdx.x * 256 + threadIdx.x;
  if (p >= npix) return;
  const T* row = delta + p * c;
  int any = 0;
  if constexpr (sizeof(T) == 4) {
    if ((c & 3) == 0) {
      const float4* r4 = reinterpret_cast<const float4*>(row);
      for (int i = 0; i < (c >> 2); ++i) {
        const float4 v = r4[i];
        any |= (fabsf(v.x) > thr) | (fabsf(v.y) > thr) | (fabsf(v.z) > thr) | (fabsf(v.w) > thr);
      }
    } else {
      for (int i = 0; i < c; ++i) any |= (fabsf(mie_ld(row, i)) > thr);
    }
  } else {
    for (int i = 0; i < c; ++i) any |= (fabsf(mie_ld(row, i)) > thr);
  }
  pixmask[p] = (uint8_t)any;
}

extern "C" int mie_mask_from_delta(const void* delta, int n, int h, int w, int c,
                                   float threshold, uint8_t* pixmask, int dtype, void* stream) {
  mie_clear_error();
  MIE_REQUIRE(delta && pixmask, MIE_ERR_INVALID_ARG, "mie_mask_from_delta: NULL pointer");
  MIE_REQUIRE(dtype == MIE_DTYPE_F32 || dtype == MIE_DTYPE_BF16, MIE_ERR_UNSUPPORTED,
              "mie_mask_from_delta: unknown delta dtype %d", dtype);
  MIE_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0, MIE_ERR_INVALID_ARG,
              "mie_mask_from_delta: sizes must be positive (n=%d h=%d w=%d c=%d)", n, h, w, c);
  MIE_REQUIRE(threshold >= 0.f, MIE_ERR_INVALID_ARG, "mie_mask_from_delta: threshold < 0");
  MIE_REQUIRE(mie_aligned(delta, 16), MIE_ERR_INVALID_ARG,
              "mie_mask_from_delta: delta must be 16-byte aligned");
  const long long npix = (long long)n * h * w;
  MIE_REQUIRE(npix < 0x7fffffffLL, MIE_ERR_CAPACITY, "mie_mask_from_delta: too many pixels");
  const unsigned blocks = (unsigned)((npix + 255) / 256);
  if (dtype == MIE_DTYPE_BF16)
    hipLaunchKernelGGL(k_mask_from_delta<mie_bf16>, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                       (const mie_bf16*)delta, npix, c, threshold, pixmask);
  else
    hipLaunchKernelGGL(k_mask_from_delta<float>, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                       (const float*)delta, npix, c, threshold, pixmask);
  return mie_check_launch("mie_mask_from_delta");
}

// ---- footprint + tile flags + ordered compaction ----------------------------
struct BuildArgs {
  const uint8_t* in;
  const uint8_t* in2;
  int n, h_in, w_in;
  int foot, k, s, p;
  uint8_t* out;
  int h_out, w_out, tiles_y, tiles_x, cap;
  int32_t* tiles;
  int32_t* stale;
  int32_t* counts;
  uint32_t* flags;
};

__device__ __forceinline__ int mask_at(const BuildArgs& a, int n, int iy, int ix) {
  if (iy < 0 || iy >= a.h_in || ix < 0 || ix >= a.w_in) return 0;
  const long long o = ((long long)n * a.h_in + iy) * a.w_in + ix;
  int v = a.in[o];
  if (a.in2) v |= a.in2[o];
  return v != 0;
}

// Source index pair of bilinear x2 (align_corners = False) with non-zero weight.
__device__ __forceinline__ void up2x_src(int o, int in_size, int& i0, int& i1) {
  const int j = o >> 1;
  if (o & 1) {
    i0 = j;
    i1 = (j + 1 < in_size) ? j + 1 : j;
  } else {
    i0 = (j > 0) ? j - 1 : 0;
    i1 = j;
  }
}

// k x k window of a conv with the window size known at compile time: every load is issued from a clamped
// address and masked afterwards, so the K * K loads of a lane are independent and go out back to back.
template <int K>
__device__ __forceinline__ int conv_window_bit(const BuildArgs& a, int n, int iy0, int ix0) {
  const uint8_t* base = a.in + (long long)n * a.h_in * a.w_in;
  const uint8_t* base2 = a.in2 ? a.in2 + (long long)n * a.h_in * a.w_in : nullptr;
  int bit = 0;
#pragma unroll
  for (int ky = 0; ky < K; ++ky) {
    const int iy = iy0 + ky;
    const bool oky = iy >= 0 && iy < a.h_in;
    const int row = (oky ? iy : 0) * a.w_in;
#pragma unroll
    for (int kx = 0; kx < K; ++kx) {
      const int ix = ix0 + kx;
      const bool ok = oky && ix >= 0 && ix < a.w_in;
      const int o = row + (ok ? ix : 0);
      int v = base[o];
      if (base2) v |= base2[o];
      bit |= ok ? v : 0;
    }
  }
  return bit != 0;
}

__device__ int footprint_bit(const BuildArgs& a, int n, int oy, int ox) {
  if (a.in == nullptr) return 1;
  int bit = 0;
  if (a.foot == MIE_FOOT_CONV) {
    const int iy0 = oy * a.s - a.p, ix0 = ox * a.s - a.p;
    if (a.k == 5) return conv_window_bit<5>(a, n, iy0, ix0);
    if (a.k == 3) return conv_window_bit<3>(a, n, iy0, ix0);
    if (a.k == 1) return conv_window_bit<1>(a, n, iy0, ix0);
    for (int ky = 0; ky < a.k; ++ky)
      for (int kx = 0; kx < a.k; ++kx) bit |= mask_at(a, n, iy0 + ky, ix0 + kx);
  } else if (a.foot == MIE_FOOT_UP2X) {
    int r0, r1, c0, c1;
    up2x_src(oy, a.h_in, r0, r1);
    up2x_src(ox, a.w_in, c0, c1);
    bit = mask_at(a, n, r0, c0) | mask_at(a, n, r0, c1) | mask_at(a, n, r1, c0) |
          mask_at(a, n, r1, c1);
  } else {  // MIE_FOOT_TCONV
    for (int ky = 0; ky < a.k; ++ky) {
      const int ty = oy + a.p - ky;
      if (ty < 0 || (ty % a.s) != 0) continue;
      for (int kx = 0; kx < a.k; ++kx) {
        const int tx = ox + a.p - kx;
        if (tx < 0 || (tx % a.s) != 0) continue;
        bit |= mask_at(a, n, ty / a.s, tx / a.s);
      }
    }
  }
  return bit;
}

// Kernel 1: one wave per output tile.  Lane = pixel of the 8x8 tile: derives its mask bit
// from the input footprint, writes the output pixel mask, and a wave ballot tells whether
// the tile holds any active pixel.
__device__ __forceinline__ bool tile_footprint(const BuildArgs& a, int tile, int lane) {
  const int tx = tile % a.tiles_x;
  const int t2 = tile / a.tiles_x;
  const int ty = t2 % a.tiles_y;
  const int n = t2 / a.tiles_y;
  const int oy = ty * MIE_TILE + (lane >> 3), ox = tx * MIE_TILE + (lane & 7);
  int bit = 0;
  if (oy < a.h_out && ox < a.w_out) {
    bit = footprint_bit(a, n, oy, ox);
    a.out[((long long)n * a.h_out + oy) * a.w_out + ox] = (uint8_t)bit;
  }
  return __ballot(bit != 0) != 0ull;
}

// flags[tile]: bit 0 = the tile holds an active pixel after this build, bit 1 = it did after the
// previous build of this tile set (what makes a tile stale).  A lane reads and writes its own word only.
__device__ __forceinline__ uint32_t next_flag(uint32_t old, bool any) { return ((old & 1u) << 1) | (any ? 1u : 0u); }

__global__ __launch_bounds__(256) void k_mask_footprint(BuildArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = blockIdx.x * 4 + wave;
  if (tile >= a.cap) return;
  const uint32_t old = a.flags[tile];          // issued ahead of the footprint's mask loads
  const bool any = tile_footprint(a, tile, lane);
  if (lane == 0) a.flags[tile] = next_flag(old, any);
}

// Ordered compaction of the tile flags into the active list (bit 0 set) and the stale list (bit 1
// set, bit 0 clear), both ascending, by a grid of COMPACT_THREADS-thread blocks without atomics or
// fences: block b owns the COMPACT_CHUNK flags [b * CHUNK, (b + 1) * CHUNK).  It first counts the two
// kinds over every flag below its chunk (16-byte loads; at most a few dozen per thread even for tens of
// thousands of tiles) -- that is its base in either list -- and then ranks its own flags: per wave a
// ballot gives 64 keep-bits, popcount below the lane the rank inside the wave, and the wave totals
// meet in LDS.  The last block also writes the two totals.
constexpr int COMPACT_THREADS = 1024;
constexpr int COMPACT_WAVES = COMPACT_THREADS / 64;
constexpr int COMPACT_ITEMS = 4;      // element j * COMPACT_THREADS + tid of the chunk, j < COMPACT_ITEMS
constexpr int COMPACT_CHUNK = COMPACT_THREADS * COMPACT_ITEMS;

__device__ __forceinline__ int wave_sum(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// flag(t) returns the flag word of tile t (from memory or, for the one-block build, from LDS).
template <typename FlagFn>
__device__ void compact_lists(const BuildArgs& a, FlagFn flag, int chunk, int base_act, int base_st, bool last,
                              int* s_tot) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  bool ka[COMPACT_ITEMS], ks[COMPACT_ITEMS];
  int ra[COMPACT_ITEMS], rs[COMPACT_ITEMS];
#pragma unroll
  for (int j = 0; j < COMPACT_ITEMS; ++j) {
    const int t = chunk * COMPACT_CHUNK + j * COMPACT_THREADS + threadIdx.x;
    const uint32_t f = (t < a.cap) ? flag(t) : 0u;
    ka[j] = (f & 1u) != 0u;
    ks[j] = (f & 3u) == 2u;
    const unsigned long long ba = __ballot(ka[j]), bs = __ballot(ks[j]);
    const unsigned long long below = (1ull << lane) - 1ull;
    ra[j] = __popcll(ba & below);
    rs[j] = __popcll(bs & below);
    if (lane == 0) {
      s_tot[j * COMPACT_WAVES + wave] = __popcll(ba);
      s_tot[COMPACT_ITEMS * COMPACT_WAVES + j * COMPACT_WAVES + wave] = __popcll(bs);
    }
  }
  __syncthreads();
  // exclusive prefix over the (j, wave) totals in element order: j major, wave minor
  int run_a = base_act, run_s = base_st;
#pragma unroll
  for (int j = 0; j < COMPACT_ITEMS; ++j) {
    int off_a = run_a, off_s = run_s;
#pragma unroll
    for (int wv = 0; wv < COMPACT_WAVES; ++wv) {
      const int ta = s_tot[j * COMPACT_WAVES + wv];
      const int tst = s_tot[COMPACT_ITEMS * COMPACT_WAVES + j * COMPACT_WAVES + wv];
      if (wv < wave) off_a += ta, off_s += tst;
      run_a += ta;
      run_s += tst;
    }
    const int t = chunk * COMPACT_CHUNK + j * COMPACT_THREADS + threadIdx.x;
    if (ka[j]) a.tiles[off_a + ra[j]] = t;
    if (ks[j]) a.stale[off_s + rs[j]] = t;
  }
  if (last && threadIdx.x == 0) {
    a.counts[MIE_CNT_ACTIVE] = run_a;
    a.counts[MIE_CNT_STALE] = run_s;
  }
}

__global__ __launch_bounds__(COMPACT_THREADS) void k_compact_tiles(BuildArgs a) {
  __shared__ int s_tot[2 * COMPACT_WAVES * COMPACT_ITEMS];
  __shared__ int s_base[2 * COMPACT_WAVES];
  const uint32_t* flags = a.flags;
  const int chunk = blockIdx.x;
  // base = number of active / stale tiles below this chunk (its start is a multiple of 4096 flags)
  int na = 0, ns = 0;
  const uint4* f4 = reinterpret_cast<const uint4*>(flags);
  const int n4 = chunk * (COMPACT_CHUNK / 4);
  for (int i = threadIdx.x; i < n4; i += COMPACT_THREADS) {
    const uint4 v = f4[i];
    na += (int)(v.x & 1u) + (int)(v.y & 1u) + (int)(v.z & 1u) + (int)(v.w & 1u);
    ns += (int)((v.x & 3u) == 2u) + (int)((v.y & 3u) == 2u) + (int)((v.z & 3u) == 2u) + (int)((v.w & 3u) == 2u);
  }
  int base_act = 0, base_st = 0;
  if (chunk > 0) {      // uniform over the block
    na = wave_sum(na);
    ns = wave_sum(ns);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) s_base[wave] = na, s_base[COMPACT_WAVES + wave] = ns;
    __syncthreads();
#pragma unroll
    for (int wv = 0; wv < COMPACT_WAVES; ++wv) base_act += s_base[wv], base_st += s_base[COMPACT_WAVES + wv];
  }
  compact_lists(a, [&](int t) { return flags[t]; }, chunk, base_act, base_st, chunk == (int)gridDim.x - 1, s_tot);
}

// Planes of at most SMALL_CAP tiles (the 33x44 plane of a 264x352 frame: 30 tiles): footprint
// and compaction in ONE block, tile flags handed over through LDS -- one launch instead of two.
constexpr int SMALL_CAP = 32;

__global__ __launch_bounds__(COMPACT_THREADS) void k_build_small(BuildArgs a) {
  __shared__ int s_tot[2 * COMPACT_WAVES * COMPACT_ITEMS];
  __shared__ unsigned s_flag[SMALL_CAP];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int tile = wave; tile < a.cap; tile += COMPACT_WAVES) {
    const uint32_t old = a.flags[tile];
    const bool any = tile_footprint(a, tile, lane);
    if (lane == 0) {
      const uint32_t f = next_flag(old, any);
      s_flag[tile] = f;
      a.flags[tile] = f;
    }
  }
  __syncthreads();
  compact_lists(a, [&](int t) { return s_flag[t]; }, 0, 0, 0, true, s_tot);
}

extern "C" int mie_build_mask_tiles(const uint8_t* in_mask, const uint8_t* in_mask2,
                                    int h_in, int w_in, int foot, int k, int stride,
                                    int pad, const mie_tileset* out, void* stream) {
  mie_clear_error();
  int rc = mie_check_tileset(out, "mie_build_mask_tiles");
  if (rc != MIE_OK) return rc;
  MIE_REQUIRE(h_in > 0 && w_in > 0, MIE_ERR_INVALID_ARG,
              "mie_build_mask_tiles: input size (%d,%d) must be positive", h_in, w_in);
  MIE_REQUIRE(in_mask != nullptr || in_mask2 == nullptr, MIE_ERR_INVALID_ARG,
              "mie_build_mask_tiles: in_mask2 given without in_mask");
  MIE_REQUIRE((long long)out->n * h_in * w_in < 0x7fffffffLL, MIE_ERR_CAPACITY,
              "mie_build_mask_tiles: more than 2^31 input pixels");
  if (foot == MIE_FOOT_CONV) {
    MIE_REQUIRE(k >= 1 && k <= 15 && stride >= 1 && stride <= 4 && pad >= 0 && pad < 16,
                MIE_ERR_UNSUPPORTED, "mie_build_mask_tiles: conv footprint k=%d stride=%d pad=%d",
                k, stride, pad);
    const int ho = (h_in + 2 * pad - k) / stride + 1, wo = (w_in + 2 * pad - k) / stride + 1;
    MIE_REQUIRE(h_in + 2 * pad >= k && w_in + 2 * pad >= k && ho == out->h && wo == out->w,
                MIE_ERR_INVALID_ARG,
                "mie_build_mask_tiles: conv output of (%d,%d) k=%d s=%d p=%d is (%d,%d), tile set is (%d,%d)",
                h_in, w_in, k, stride, pad, ho, wo, out->h, out->w);
  } else if (foot == MIE_FOOT_UP2X) {
    MIE_REQUIRE(out->h == 2 * h_in && out->w == 2 * w_in, MIE_ERR_INVALID_ARG,
                "mie_build_mask_tiles: up2x of (%d,%d) is not (%d,%d)", h_in, w_in, out->h, out->w);
  } else if (foot == MIE_FOOT_TCONV) {
    MIE_REQUIRE(k >= 1 && k <= 15 && stride >= 1 && stride <= 4 && pad >= 0 && pad < 16,
                MIE_ERR_UNSUPPORTED, "mie_build_mask_tiles: tconv footprint k=%d stride=%d pad=%d",
                k, stride, pad);
    const int hmin = (h_in - 1) * stride - 2 * pad + k, wmin = (w_in - 1) * stride - 2 * pad + k;
    MIE_REQUIRE(out->h >= hmin && out->h < hmin + stride && out->w >= wmin && out->w < wmin + stride,
                MIE_ERR_INVALID_ARG,
                "mie_build_mask_tiles: tconv output (%d,%d) not in [(%d,%d), +stride)", out->h,
                out->w, hmin, wmin);
  } else {
    MIE_REQUIRE(false, MIE_ERR_UNSUPPORTED, "mie_build_mask_tiles: unknown footprint %d", foot);
  }
  // A lane reads the mask bytes of its footprint while other lanes write theirs: only the 1x1 stride-1
  // identity footprint (own pixel in, own pixel out) may be built in place.
  const bool identity = foot == MIE_FOOT_CONV && k == 1 && stride == 1 && pad == 0;
  MIE_REQUIRE(identity || ((const uint8_t*)out->pixmask != in_mask && (const uint8_t*)out->pixmask != in_mask2),
              MIE_ERR_INVALID_ARG,
              "mie_build_mask_tiles: out->pixmask aliases an input mask (allowed for the 1x1 stride-1 footprint only)");
  BuildArgs a;
  a.in = in_mask; a.in2 = in_mask2;
  a.n = out->n; a.h_in = h_in; a.w_in = w_in;
  a.foot = foot; a.k = k; a.s = stride; a.p = pad;
  a.out = out->pixmask; a.h_out = out->h; a.w_out = out->w;
  a.tiles_y = mie_div_up(out->h, MIE_TILE); a.tiles_x = mie_div_up(out->w, MIE_TILE);
  a.cap = mie_tile_capacity(out->n, out->h, out->w);
  a.tiles = out->tiles; a.stale = out->stale; a.counts = out->counts; a.flags = out->flags;
  if (a.cap <= SMALL_CAP) {
    hipLaunchKernelGGL(k_build_small, dim3(1), dim3(COMPACT_THREADS), 0, (hipStream_t)stream, a);
    return mie_check_launch("mie_build_mask_tiles");
  }
  const unsigned blocks = (unsigned)mie_div_up(a.cap, 4);
  hipLaunchKernelGGL(k_mask_footprint, dim3(blocks), dim3(256), 0, (hipStream_t)stream, a);
  rc = mie_check_launch("mie_build_mask_tiles");
  if (rc != MIE_OK) return rc;
  hipLaunchKernelGGL(k_compact_tiles, dim3((unsigned)mie_div_up(a.cap, COMPACT_CHUNK)), dim3(COMPACT_THREADS), 0,
                     (hipStream_t)stream, a);
  return mie_check_launch("mie_build_mask_tiles");
}
