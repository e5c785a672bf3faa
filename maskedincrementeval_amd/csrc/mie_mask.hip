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

// Few channels that are no multiple of 4 (a network's input: 5 event bins): a pixel's row is 10 or 20 bytes, and one
// thread per pixel reads it in 2- or 4-byte pieces at a stride of that many bytes.  Here a wave takes the 64 * c elements
// of its 64 pixels as ONE contiguous span in 16-byte loads (the span starts at a multiple of 64 * c * sizeof(T) bytes,
// so every load is aligned), tests its elements and marks their pixels -- element e of the span belongs to pixel e / c
// -- in LDS; lane p then writes the byte of pixel p.  8x480x640x5 bf16: 35 -> 10 us on its own.
constexpr int MFD_SMALL_C = 16;      // channels up to which this form is taken
template <typename T>
__global__ __launch_bounds__(256) void k_mask_from_delta_span(
    const T* __restrict__ delta, long long npix, int c, float thr, uint8_t* __restrict__ pixmask) {
  constexpr int EPL = 16 / (int)sizeof(T);      // elements per 16-byte load
  __shared__ unsigned s_any[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long long p0 = ((long long)blockIdx.x * 4 + wave) * 64;      // first pixel of this wave
  s_any[wave][lane] = 0u;
  if (p0 < npix) {      // uniform over the wave
    const long long total = npix * c;                 // elements of the whole delta
    const long long e0 = p0 * c;                      // first element of the span
    const int span = 64 * c;                          // elements of a full span
    const unsigned inv_c = (65536u + (unsigned)c - 1u) / (unsigned)c;      // e / c for e < 64 * 16, c <= 16
    for (int ch = lane; ch * EPL < span; ch += 64) {
      const long long e = e0 + (long long)ch * EPL;
      if (e >= total) break;
      float f[EPL];
      if (e + EPL <= total) {
        const float4 raw = *reinterpret_cast<const float4*>(delta + e);
        if constexpr (sizeof(T) == 4) {
          f[0] = raw.x; f[1] = raw.y; f[2] = raw.z; f[3] = raw.w;
        } else {
          const unsigned w4[4] = {__float_as_uint(raw.x), __float_as_uint(raw.y), __float_as_uint(raw.z), __float_as_uint(raw.w)};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            f[2 * j] = __uint_as_float(w4[j] << 16);
            f[2 * j + 1] = __uint_as_float(w4[j] & 0xffff0000u);
          }
        }
      } else {      // the last load of the delta would run past its end
#pragma unroll
        for (int j = 0; j < EPL; ++j) f[j] = (e + j < total) ? mie_ld(delta, e + j) : 0.f;
      }
#pragma unroll
      for (int j = 0; j < EPL; ++j) {
        if (fabsf(f[j]) > thr) {
          const unsigned le = (unsigned)(ch * EPL + j);      // element of the span
          s_any[wave][(le * inv_c) >> 16] = 1u;
        }
      }
    }
  }
  __syncthreads();
  if (p0 + lane < npix) pixmask[p0 + lane] = (uint8_t)s_any[wave][lane];
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
  const bool span = (c & 3) != 0 && c <= MFD_SMALL_C;
  if (dtype == MIE_DTYPE_BF16) {
    if (span)
      hipLaunchKernelGGL(k_mask_from_delta_span<mie_bf16>, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                         (const mie_bf16*)delta, npix, c, threshold, pixmask);
    else
      hipLaunchKernelGGL(k_mask_from_delta<mie_bf16>, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                         (const mie_bf16*)delta, npix, c, threshold, pixmask);
  } else {
    if (span)
      hipLaunchKernelGGL(k_mask_from_delta_span<float>, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                         (const float*)delta, npix, c, threshold, pixmask);
    else
      hipLaunchKernelGGL(k_mask_from_delta<float>, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                         (const float*)delta, npix, c, threshold, pixmask);
  }
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

// One chunk of the compaction of a tile set: block `chunk` of `nchunks`.
__device__ void compact_chunk(const BuildArgs& a, int chunk, int nchunks, int* s_tot, int* s_base) {
  const uint32_t* flags = a.flags;
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
  compact_lists(a, [&](int t) { return flags[t]; }, chunk, base_act, base_st, chunk == nchunks - 1, s_tot);
}

__global__ __launch_bounds__(COMPACT_THREADS) void k_compact_tiles(BuildArgs a) {
  __shared__ int s_tot[2 * COMPACT_WAVES * COMPACT_ITEMS];
  __shared__ int s_base[2 * COMPACT_WAVES];
  compact_chunk(a, blockIdx.x, (int)gridDim.x, s_tot, s_base);
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

// ---- one launch for planes of up to TICKET_CAP tiles ----------------------------------------------
// The footprint kernel's workgroups take a ticket from counts[MIE_CNT_TICKET] when their flags are written; the one
// that draws the last ticket puts the counter back to zero and ranks the two lists from the flags of all of them.
// Nobody waits for anybody: every other workgroup has left by then.  The lists are what k_compact_tiles writes.
// Flags are stored and, by the last workgroup, loaded as device-scope atomics, which go through to the level the
// XCDs share; a workgroup waits for its flag stores to complete before it draws its ticket.  (A device-scope
// release / acquire fence pair would order ordinary stores as well, but it writes back and invalidates the whole L2
// of the XCD -- with a step's deltas in it that cost 8 us per build, more than the launch it saves.)  The pixel masks
// are ordinary stores: nothing in the kernel reads another workgroup's.
constexpr int TICKET_CAP = 4096;
constexpr int TICKET_THREADS = 256;
constexpr int TICKET_ITEMS = TICKET_CAP / TICKET_THREADS;      // consecutive flags per thread

__device__ __forceinline__ void store_flag(uint32_t* flags, int tile, uint32_t f) {
  __hip_atomic_store(flags + tile, f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// true in exactly one workgroup of the grid: the one whose ticket is the last
__device__ __forceinline__ bool last_workgroup(int32_t* counts, int* s_last) {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");      // this thread's flag stores have completed
  __syncthreads();
  if (threadIdx.x == 0) {
    const int t = __hip_atomic_fetch_add(&counts[MIE_CNT_TICKET], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool last = t == (int)gridDim.x - 1;
    if (last) __hip_atomic_store(&counts[MIE_CNT_TICKET], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // all drawn
    *s_last = last ? 1 : 0;
  }
  __syncthreads();
  return *s_last != 0;
}

// the two lists of a set of at most TICKET_CAP tiles, by the first TICKET_THREADS threads of one workgroup (all of its
// threads call)
__device__ void compact_by_one(const BuildArgs& a, int* s_w) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint32_t f[TICKET_ITEMS];
  int na = 0, ns = 0;
#pragma unroll
  for (int j = 0; j < TICKET_ITEMS; ++j) {
    const int t = tid * TICKET_ITEMS + j;
    f[j] = (tid < TICKET_THREADS && t < a.cap) ? __hip_atomic_load(a.flags + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
    na += (int)(f[j] & 1u);
    ns += (int)((f[j] & 3u) == 2u);
  }
  // exclusive prefix over the threads: inside the wave by shuffles, wave totals through LDS
  int ia = na, is = ns;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int ua = __shfl_up(ia, o), us = __shfl_up(is, o);
    if (lane >= o) ia += ua, is += us;
  }
  if (lane == 63 && wave < TICKET_THREADS / 64) s_w[wave] = ia, s_w[4 + wave] = is;
  __syncthreads();
  if (tid >= TICKET_THREADS) return;      // a wider workgroup: its other waves only meet the barrier
  int pa = ia - na, ps = is - ns, ta = 0, tst = 0;
#pragma unroll
  for (int wv = 0; wv < TICKET_THREADS / 64; ++wv) {
    if (wv < wave) pa += s_w[wv], ps += s_w[4 + wv];
    ta += s_w[wv];
    tst += s_w[4 + wv];
  }
#pragma unroll
  for (int j = 0; j < TICKET_ITEMS; ++j) {
    const int t = tid * TICKET_ITEMS + j;
    if (f[j] & 1u) a.tiles[pa++] = t;
    if ((f[j] & 3u) == 2u) a.stale[ps++] = t;
  }
  if (tid == 0) {
    a.counts[MIE_CNT_ACTIVE] = ta;
    a.counts[MIE_CNT_STALE] = tst;
  }
}

// k_mask_footprint + k_compact_tiles for sets of up to TICKET_CAP tiles
__global__ __launch_bounds__(TICKET_THREADS) void k_mask_footprint_lists(BuildArgs a) {
  __shared__ int s_w[8];
  __shared__ int s_last;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = blockIdx.x * 4 + wave;
  if (tile < a.cap) {
    const uint32_t old = a.flags[tile];
    const bool any = tile_footprint(a, tile, lane);
    if (lane == 0) store_flag(a.flags, tile, next_flag(old, any));
  }
  if (last_workgroup(a.counts, &s_last)) compact_by_one(a, s_w);
}

// ---- threshold mask + footprint (+ lists) in one launch -------------------------------------------
// What mie_mask_from_delta followed by mie_build_mask_tiles (conv footprint) leave, for the thresholded masks of
// the lossy networks: one workgroup per output tile tests the input pixels of its tile's windows against the
// threshold itself, straight from the delta, keeps the bits in LDS, writes the bytes of the input pixels it owns (the
// 8s x 8s block under its tile; the last row / column of tiles owns through the plane's edge) and forms the footprint
// from LDS.  Pixels in the halo of a window are tested by up to four workgroups; a delta plane of these networks is
// at most a few MB and the launch is bound by latency -- so the test is a flat loop over (pixel, 4-channel group)
// pairs with eight loads in flight per thread and no exchange between lanes (a hit sets the pixel's byte in LDS).
struct ThrArgs {
  BuildArgs b;          // b.in is unused (the mask comes from delta); b.in2 as in mie_build_mask_tiles
  const void* delta;
  uint8_t* thr_mask;    // [n, h_in, w_in]: the thresholded mask, as mie_mask_from_delta writes it
  int c;
  int vec_shift;        // log2(c / 4) when c / 4 is a power of two, else -1
  float thr;
  int lists;            // 1: the last workgroup ranks the lists
};
constexpr int THR_EDGE = 24;      // largest region edge: 7 * s + k (+ the rows no window reaches)
constexpr int THR_UNROLL = 8;
constexpr int TICKET_MAX_WGS = 128;      // more workgroups than this queue up at the ticket counter: two launches then

template <typename T>
__global__ __launch_bounds__(1024) void k_build_thresholded(ThrArgs a) {
  __shared__ uint8_t s_in[THR_EDGE * THR_EDGE];
  __shared__ int s_w[8];
  __shared__ int s_last;
  const BuildArgs& b = a.b;
  const int tid = threadIdx.x, nthr = blockDim.x, lane = tid & 63;
  const int tile = blockIdx.x;                    // the grid is one workgroup per tile
  const int tx = tile % b.tiles_x, t2 = tile / b.tiles_x, ty = t2 % b.tiles_y, n = t2 / b.tiles_y;
  uint32_t old = 0;
  if (tid == 0) old = b.flags[tile];
  const int r0 = ty * MIE_TILE * b.s - b.p, c0 = tx * MIE_TILE * b.s - b.p;
  const int own_r0 = ty * MIE_TILE * b.s, own_c0 = tx * MIE_TILE * b.s;
  const int own_r1 = (ty == b.tiles_y - 1) ? b.h_in : own_r0 + MIE_TILE * b.s;
  const int own_c1 = (tx == b.tiles_x - 1) ? b.w_in : own_c0 + MIE_TILE * b.s;
  const int win = 7 * b.s + b.k;
  const int rows = max(r0 + win, own_r1) - r0, cols = max(c0 + win, own_c1) - c0;
  const int npx = rows * cols;
  const unsigned col_magic = (65536u + (unsigned)cols - 1u) / (unsigned)cols;      // p / cols for p < 576, cols <= 24
  const T* plane = static_cast<const T*>(a.delta) + (long long)n * b.h_in * b.w_in * a.c;
  for (int i = tid; i < npx; i += nthr) s_in[i] = 0;
  __syncthreads();
  if ((a.c & 3) == 0) {
    const int nvec = a.c >> 2, total = npx * nvec;
    for (int base = tid; base < total; base += THR_UNROLL * nthr) {
      float4 v[THR_UNROLL];
      int pp[THR_UNROLL];
#pragma unroll
      for (int u = 0; u < THR_UNROLL; ++u) {
        const int idx = base + u * nthr;
        const int p = a.vec_shift >= 0 ? (idx >> a.vec_shift) : idx / nvec;
        const int q = idx - p * nvec;
        const int ry = (int)(((unsigned)p * col_magic) >> 16), rx = p - ry * cols;
        const int iy = r0 + ry, ix = c0 + rx;
        const bool inside = idx < total && iy >= 0 && iy < b.h_in && ix >= 0 && ix < b.w_in;
        pp[u] = inside ? p : -1;
        // every load goes out, from a clamped address: eight independent loads, no branch between them
        v[u] = mie_ld4(plane + (inside ? ((long long)iy * b.w_in + ix) * a.c + 4 * q : 0ll), 0);
      }
#pragma unroll
      for (int u = 0; u < THR_UNROLL; ++u) {
        const bool hit = (fabsf(v[u].x) > a.thr) | (fabsf(v[u].y) > a.thr) | (fabsf(v[u].z) > a.thr) | (fabsf(v[u].w) > a.thr);
        if (pp[u] >= 0 && hit) s_in[pp[u]] = 1;
      }
    }
  } else {      // channel counts that are no multiple of 4 (a network's input): one thread per pixel
    for (int p = tid; p < npx; p += nthr) {
      const int ry = (int)(((unsigned)p * col_magic) >> 16), rx = p - ry * cols;
      const int iy = r0 + ry, ix = c0 + rx;
      if (iy < 0 || iy >= b.h_in || ix < 0 || ix >= b.w_in) continue;
      const T* row = plane + ((long long)iy * b.w_in + ix) * a.c;
      int any = 0;
      for (int i = 0; i < a.c; ++i) any |= (fabsf(mie_ld(row, i)) > a.thr);
      if (any) s_in[p] = 1;
    }
  }
  __syncthreads();
  for (int p = tid; p < npx; p += nthr) {
    const int ry = (int)(((unsigned)p * col_magic) >> 16), rx = p - ry * cols;
    const int iy = r0 + ry, ix = c0 + rx;
    if (iy >= own_r0 && iy < min(own_r1, b.h_in) && ix >= own_c0 && ix < min(own_c1, b.w_in))
      a.thr_mask[((long long)n * b.h_in + iy) * b.w_in + ix] = s_in[p];
  }
  if (tid < 64) {
    const int py = lane >> 3, px = lane & 7;
    const int oy = ty * MIE_TILE + py, ox = tx * MIE_TILE + px;
    int bit = 0;
    if (oy < b.h_out && ox < b.w_out) {
      for (int ky = 0; ky < b.k; ++ky)
        for (int kx = 0; kx < b.k; ++kx) bit |= s_in[(py * b.s + ky) * cols + px * b.s + kx];
      if (b.in2) {
        const uint8_t* m2 = b.in2 + (long long)n * b.h_in * b.w_in;
        for (int ky = 0; ky < b.k; ++ky) {
          const int iy = oy * b.s - b.p + ky;
          if (iy < 0 || iy >= b.h_in) continue;
          for (int kx = 0; kx < b.k; ++kx) {
            const int ix = ox * b.s - b.p + kx;
            if (ix >= 0 && ix < b.w_in) bit |= m2[iy * b.w_in + ix];
          }
        }
      }
      bit = bit != 0;
      b.out[((long long)n * b.h_out + oy) * b.w_out + ox] = (uint8_t)bit;
    }
    const bool any = __ballot(bit != 0) != 0ull;
    if (lane == 0) {
      if (a.lists) store_flag(b.flags, tile, next_flag(old, any));
      else b.flags[tile] = next_flag(old, any);
    }
  }
  if (a.lists && last_workgroup(b.counts, &s_last)) compact_by_one(b, s_w);
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
  static const int ticket_wgs = [] { const char* e = getenv("MIE_BUILD_TICKET"); return e ? atoi(e) : TICKET_MAX_WGS; }();   // tuning knob
  if ((int)blocks <= ticket_wgs && a.cap <= TICKET_CAP) {
    hipLaunchKernelGGL(k_mask_footprint_lists, dim3(blocks), dim3(TICKET_THREADS), 0, (hipStream_t)stream, a);
    return mie_check_launch("mie_build_mask_tiles");
  }
  hipLaunchKernelGGL(k_mask_footprint, dim3(blocks), dim3(256), 0, (hipStream_t)stream, a);
  rc = mie_check_launch("mie_build_mask_tiles");
  if (rc != MIE_OK) return rc;
  hipLaunchKernelGGL(k_compact_tiles, dim3((unsigned)mie_div_up(a.cap, COMPACT_CHUNK)), dim3(COMPACT_THREADS), 0,
                     (hipStream_t)stream, a);
  return mie_check_launch("mie_build_mask_tiles");
}

extern "C" int mie_build_mask_tiles_thresholded(const void* delta, int c, int dtype, float threshold, uint8_t* thr_mask,
                                                const uint8_t* in_mask2, int h_in, int w_in, int k, int stride, int pad,
                                                const mie_tileset* out, void* stream) {
  const char* who = "mie_build_mask_tiles_thresholded";
  mie_clear_error();
  int rc = mie_check_tileset(out, who);
  if (rc != MIE_OK) return rc;
  MIE_REQUIRE(delta && thr_mask, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(dtype == MIE_DTYPE_F32 || dtype == MIE_DTYPE_BF16, MIE_ERR_UNSUPPORTED, "%s: unknown delta dtype %d", who, dtype);
  MIE_REQUIRE(h_in > 0 && w_in > 0 && c > 0, MIE_ERR_INVALID_ARG, "%s: sizes must be positive (h=%d w=%d c=%d)", who, h_in, w_in, c);
  MIE_REQUIRE(threshold >= 0.f, MIE_ERR_INVALID_ARG, "%s: threshold < 0", who);
  MIE_REQUIRE(mie_aligned(delta, 16), MIE_ERR_INVALID_ARG, "%s: delta must be 16-byte aligned", who);
  MIE_REQUIRE((long long)out->n * h_in * w_in < 0x7fffffffLL, MIE_ERR_CAPACITY, "%s: more than 2^31 input pixels", who);
  MIE_REQUIRE(k >= 1 && stride >= 1 && pad >= 0, MIE_ERR_UNSUPPORTED, "%s: conv footprint k=%d stride=%d pad=%d", who, k, stride, pad);
  // a workgroup owns the input block under its tile and must find it inside its tile's windows
  MIE_REQUIRE(stride + pad <= k && 7 * stride + k + (stride - 1 - pad > 0 ? stride - 1 - pad : 0) <= THR_EDGE,
              MIE_ERR_UNSUPPORTED, "%s: no one-launch form for k=%d stride=%d pad=%d (mie_mask_from_delta + mie_build_mask_tiles take it)",
              who, k, stride, pad);
  const int ho = (h_in + 2 * pad - k) / stride + 1, wo = (w_in + 2 * pad - k) / stride + 1;
  MIE_REQUIRE(h_in + 2 * pad >= k && w_in + 2 * pad >= k && ho == out->h && wo == out->w, MIE_ERR_INVALID_ARG,
              "%s: conv output of (%d,%d) k=%d s=%d p=%d is (%d,%d), tile set is (%d,%d)", who, h_in, w_in, k, stride, pad,
              ho, wo, out->h, out->w);
  MIE_REQUIRE(thr_mask != out->pixmask && in_mask2 != out->pixmask && in_mask2 != thr_mask, MIE_ERR_INVALID_ARG,
              "%s: thr_mask, in_mask2 and out->pixmask must be three buffers", who);
  ThrArgs a;
  memset(&a, 0, sizeof(a));
  BuildArgs& b = a.b;
  b.in = nullptr; b.in2 = in_mask2;
  b.n = out->n; b.h_in = h_in; b.w_in = w_in;
  b.foot = MIE_FOOT_CONV; b.k = k; b.s = stride; b.p = pad;
  b.out = out->pixmask; b.h_out = out->h; b.w_out = out->w;
  b.tiles_y = mie_div_up(out->h, MIE_TILE); b.tiles_x = mie_div_up(out->w, MIE_TILE);
  b.cap = mie_tile_capacity(out->n, out->h, out->w);
  b.tiles = out->tiles; b.stale = out->stale; b.counts = out->counts; b.flags = out->flags;
  a.delta = delta; a.thr_mask = thr_mask; a.c = c; a.thr = threshold;
  a.vec_shift = -1;
  if ((c & 3) == 0 && ((c >> 2) & ((c >> 2) - 1)) == 0)
    for (a.vec_shift = 0; (1 << a.vec_shift) < (c >> 2); ++a.vec_shift) {}
  static const int ticket_wgs = [] { const char* e = getenv("MIE_BUILD_TICKET"); return e ? atoi(e) : TICKET_MAX_WGS; }();   // tuning knob
  a.lists = b.cap <= ticket_wgs && b.cap <= TICKET_CAP ? 1 : 0;
  // deep planes of few tiles (fewer workgroups than CUs): more threads per tile, so that a thread's loads go out in one
  // round (thresholded 264x352 frame, cap 0 / 128 / 512 / 2048: 0.504 / 0.485 / 0.490 / 0.501 ms)
  static const int wide_cap = [] { const char* e = getenv("MIE_THR_WIDE_CAP"); return e ? atoi(e) : 128; }();      // tuning knob
  const int threads = (b.cap <= wide_cap && (long long)(7 * stride + k) * (7 * stride + k) * (c / 4) > THR_UNROLL * 256) ? 1024 : 256;
  if (dtype == MIE_DTYPE_BF16)
    hipLaunchKernelGGL(k_build_thresholded<mie_bf16>, dim3((unsigned)b.cap), dim3(threads), 0, (hipStream_t)stream, a);
  else
    hipLaunchKernelGGL(k_build_thresholded<float>, dim3((unsigned)b.cap), dim3(threads), 0, (hipStream_t)stream, a);
  rc = mie_check_launch(who);
  if (rc != MIE_OK || a.lists) return rc;
  hipLaunchKernelGGL(k_compact_tiles, dim3((unsigned)mie_div_up(b.cap, COMPACT_CHUNK)), dim3(COMPACT_THREADS), 0,
                     (hipStream_t)stream, b);
  return mie_check_launch(who);
}

// ---- every tile set of a network in two launches ------------------------------------------------
// mie_build_mask_plan runs a sequence of mie_build_mask_tiles calls -- every structural mask of a network is a chain
// of footprints of the input pixel mask -- as two kernels.  In the first, a workgroup keeps the pixel masks of one
// sample's chain as BITMAPS in LDS (a 264x352 plane is 11.6 KB): a footprint is then a handful of word operations
// per 32 pixels -- the window of a conv is the OR of the rows it covers, shifted left and right (stride 2: the even
// bits of that, compressed); bilinear x2 and the stride-2 transposed conv interleave two such ORs bit by bit --
// instead of k*k byte loads per pixel, and no launch or memory round trip separates one mask of the chain from the
// next.  That part is so cheap that several workgroups per sample each walk the whole chain on their own and share
// only what goes to memory: of every set's pixel mask (bytes, 16 per store where the rows allow it) and tile flags a
// workgroup writes its slice, so the stores of a large plane do not queue up behind one CU.  The second kernel
// ranks the lists of all sets, one block per 4096 tiles of each (as k_compact_tiles).  Slots of LDS are handed out
// on the host by lifetime (a mask is dropped after its last reader).
namespace {

constexpr int PLAN_THREADS = COMPACT_THREADS;
constexpr int PLAN_MAX_SHARES = 64;                    // workgroups per sample
constexpr int PLAN_PIXELS_PER_SHARE = 8192;            // of the plan's largest plane: 128 tiles, so a thread owns at most one
constexpr int PLAN_STEP_LOAD = 0, PLAN_STEP_FOOT = 1;
constexpr int PLAN_IN_NONE = -1, PLAN_IN_ALL = -2;

struct PlanStep {
  int kind;                 // PLAN_STEP_LOAD: bytes -> bitmap; PLAN_STEP_FOOT: footprint of one or two bitmaps
  int in1, in2;             // LDS word offsets of the input bitmaps (PLAN_IN_*)
  int out;                  // LDS word offset of the bitmap this step makes
  int h_in, w_in, h_out, w_out;
  int geom;                 // foot | k << 8 | stride << 16 | pad << 24
  int flag_off, flag_cnt;   // this step's part of the workgroup's flag area in LDS: first word, words
  int key;                  // which specialised form of the footprint runs (PLAN_KEY_*), chosen on the host
  unsigned m_words, m_units, m_tiles;   // plan_magic of the words per row, the 16-pixel units per row, the tiles per row
  int pad_;
  const uint8_t* ext;       // LOAD: the mask in memory, [n, h_out, w_out]
  uint8_t* pixmask;
  uint32_t* flags;
};

struct PlanArgs {
  int n_steps, n, flag_words, pad1_;
#ifdef MIE_PLAN_PROFILE
  int* dbg;                // measurement builds only: 2 ticks per step
#endif
  PlanStep st[MIE_PLAN_MAX_STEPS];
};
constexpr int PLAN_HEAD = MIE_PLAN_MAX_STEPS * (int)(sizeof(PlanStep) / 4);     // words of LDS in front of the bitmaps: the steps

// a step's fields, read from LDS (the same address in every lane), as scalars
__device__ __forceinline__ int plan_uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
template <typename P>
__device__ __forceinline__ P* plan_uni(P* p) {
  const unsigned long long v = reinterpret_cast<unsigned long long>(p);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
  return reinterpret_cast<P*>(((unsigned long long)hi << 32) | lo);
}
__device__ __forceinline__ PlanStep plan_uni(const PlanStep& s) {
  PlanStep u;
  u.kind = plan_uni(s.kind); u.in1 = plan_uni(s.in1); u.in2 = plan_uni(s.in2); u.out = plan_uni(s.out);
  u.h_in = plan_uni(s.h_in); u.w_in = plan_uni(s.w_in); u.h_out = plan_uni(s.h_out); u.w_out = plan_uni(s.w_out);
  u.geom = plan_uni(s.geom); u.flag_off = plan_uni(s.flag_off); u.flag_cnt = plan_uni(s.flag_cnt); u.key = plan_uni(s.key);
  u.m_words = (unsigned)plan_uni((int)s.m_words); u.m_units = (unsigned)plan_uni((int)s.m_units);
  u.m_tiles = (unsigned)plan_uni((int)s.m_tiles); u.pad_ = 0;
  u.ext = plan_uni(s.ext); u.pixmask = plan_uni(s.pixmask); u.flags = plan_uni(s.flags);
  return u;
}

// bit x of the result = bit (x + t) of the row whose words around the current one are prev, cur, next (|t| < 32):
// 32 bits out of the middle of two adjacent words (v_alignbit_b32), no branch on the sign of t
__device__ __forceinline__ uint32_t plan_shift(uint32_t prev, uint32_t cur, uint32_t next, int t) {
  const uint32_t hi = t >= 0 ? next : cur, lo = t >= 0 ? cur : prev;
  return __builtin_amdgcn_alignbit(hi, lo, (uint32_t)t & 31u);
}
// bits 0, 2, 4, ... of x packed into the low half
__device__ __forceinline__ uint32_t plan_even_bits(uint32_t x) {
  x &= 0x55555555u;
  x = (x | (x >> 1)) & 0x33333333u;
  x = (x | (x >> 2)) & 0x0f0f0f0fu;
  x = (x | (x >> 4)) & 0x00ff00ffu;
  x = (x | (x >> 8)) & 0x0000ffffu;
  return x;
}
// bit i of the low half of x moved to bit 2i
__device__ __forceinline__ uint32_t plan_spread(uint32_t x) {
  x &= 0x0000ffffu;
  x = (x | (x << 8)) & 0x00ff00ffu;
  x = (x | (x << 4)) & 0x0f0f0f0fu;
  x = (x | (x << 2)) & 0x33333333u;
  x = (x | (x << 1)) & 0x55555555u;
  return x;
}
// four mask bytes -> four bits (a byte counts when it is not zero)
__device__ __forceinline__ uint32_t plan_nibble(uint32_t v) {
  const uint32_t t = (v | ((v | 0x80808080u) - 0x01010101u)) & 0x80808080u;     // bit 7 of every non-zero byte
  return ((t >> 7) & 1u) | ((t >> 14) & 2u) | ((t >> 21) & 4u) | ((t >> 28) & 8u);
}
// four bits -> four bytes of 0 / 1
__device__ __forceinline__ uint32_t plan_bytes(uint32_t nib) {
  return (nib & 1u) | ((nib & 2u) << 7) | ((nib & 4u) << 14) | ((nib & 8u) << 21);
}

// The input of a step: one bitmap, or (TWO) the OR of two.  Every load below goes out unconditionally from a clamped
// address and is masked afterwards, so that the loads of a whole window are in flight together instead of one row
// after the other.
template <bool TWO>
struct PlanRowAcc {
  const uint32_t* b1;
  const uint32_t* b2;
  int ww, h;
  __device__ __forceinline__ uint32_t at(int y, int j) const {
    return TWO ? (b1[y * ww + j] | b2[y * ww + j]) : b1[y * ww + j];
  }
  // row y if it exists, else all zeros: (clamped row, mask)
  __device__ __forceinline__ int row(int y, uint32_t& m) const {
    const bool ok = y >= 0 && y < h;
    m = ok ? 0xffffffffu : 0u;
    return ok ? y : 0;
  }
};

// One output word of a footprint step: pixels 32*j .. 32*j+31 of row oy.  K = 0: kernel size read at run time.
struct PlanGeom { int k, p; };
template <int FOOT, int K, int S, bool TWO>
__device__ __forceinline__ uint32_t plan_foot_word(const PlanGeom& g, const PlanRowAcc<TWO>& in, int oy, int j) {
  // kernel size and padding: compile-time constants for the common footprints (K > 0: "same" padding K / 2)
  const PlanGeom s = {K > 0 ? K : g.k, K > 0 ? K / 2 : g.p};
  const int k = s.k;
  const int ww = in.ww, h = in.h;
  if (FOOT == MIE_FOOT_CONV && S == 1) {
    const int lo = -s.p;
    const bool okp = j > 0, okc = j < ww, okn = j + 1 < ww;
    const int jp = okp ? j - 1 : 0, jc = okc ? j : 0, jn = okn ? j + 1 : 0;
    uint32_t vp = 0u, vc = 0u, vn = 0u;
#pragma unroll
    for (int ky = 0; ky < k; ++ky) {
      uint32_t m;
      const int iy = in.row(oy - s.p + ky, m);
      vp |= in.at(iy, jp) & m;
      vc |= in.at(iy, jc) & m;
      vn |= in.at(iy, jn) & m;
    }
    vp = okp ? vp : 0u; vc = okc ? vc : 0u; vn = okn ? vn : 0u;
    uint32_t r = 0u;
#pragma unroll
    for (int t = 0; t < k; ++t) r |= plan_shift(vp, vc, vn, lo + t);
    return r;
  }
  if (FOOT == MIE_FOOT_CONV) {
    // stride 2: the window OR at input positions 64*j .. 64*j+63, of which the even ones are the outputs
    const int lo = -s.p;
    const int j0 = 2 * j - 1;
    bool ok[4];
    int jj[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      ok[q] = j0 + q >= 0 && j0 + q < ww;
      jj[q] = ok[q] ? j0 + q : 0;
    }
    uint32_t v[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int ky = 0; ky < k; ++ky) {
      uint32_t m;
      const int iy = in.row(2 * oy - s.p + ky, m);
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] |= in.at(iy, jj[q]) & m;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) v[q] = ok[q] ? v[q] : 0u;
    uint32_t d0 = 0u, d1 = 0u;
#pragma unroll
    for (int t = 0; t < k; ++t) {
      d0 |= plan_shift(v[0], v[1], v[2], lo + t);
      d1 |= plan_shift(v[1], v[2], v[3], lo + t);
    }
    return plan_even_bits(d0) | (plan_even_bits(d1) << 16);
  }
  const int js = j >> 1, sh = 16 * (j & 1);
  const bool okp = js > 0, okc = js < ww, okn = js + 1 < ww;
  const int jp = okp ? js - 1 : 0, jc = okc ? js : 0, jn = okn ? js + 1 : 0;
  uint32_t vp = 0u, vc = 0u, vn = 0u;
  if (FOOT == MIE_FOOT_UP2X) {
    // out[2m] = in[m-1] | in[m], out[2m+1] = in[m] | in[m+1], rows and columns alike (clamping at the border adds
    // nothing: the clamped neighbour is the pixel itself)
    int r0, r1;
    up2x_src(oy, h, r0, r1);
    vp = in.at(r0, jp) | in.at(r1, jp);
    vc = in.at(r0, jc) | in.at(r1, jc);
    vn = in.at(r0, jn) | in.at(r1, jn);
    vp = okp ? vp : 0u; vc = okc ? vc : 0u; vn = okn ? vn : 0u;
    const uint32_t ev = vc | plan_shift(vp, vc, vn, -1), od = vc | plan_shift(vp, vc, vn, 1);
    return plan_spread(ev >> sh) | (plan_spread(od >> sh) << 1);
  }
  // MIE_FOOT_TCONV, stride 2: output 2m + e sees input m + (e + p - kk) / 2 for the taps kk with e + p - kk even
  const int e = oy & 1, m_ = oy >> 1;
#pragma unroll
  for (int ky = 0; ky < k; ++ky) {
    const int d2 = e + s.p - ky;
    uint32_t m;
    const int iy = in.row(m_ + (d2 >> 1), m);
    m = (d2 & 1) ? 0u : m;
    vp |= in.at(iy, jp) & m;
    vc |= in.at(iy, jc) & m;
    vn |= in.at(iy, jn) & m;
  }
  vp = okp ? vp : 0u; vc = okc ? vc : 0u; vn = okn ? vn : 0u;
  uint32_t ev = 0u, od = 0u;
#pragma unroll
  for (int kx = 0; kx < k; ++kx) {
    const int d2 = s.p - kx;
    if (d2 & 1) od |= plan_shift(vp, vc, vn, (d2 + 1) >> 1);
    else ev |= plan_shift(vp, vc, vn, d2 >> 1);
  }
  return plan_spread(ev >> sh) | (plan_spread(od >> sh) << 1);
}

// floor(a / d) with m = plan_magic(d) = ceil(2^32 / d) worked out on the host: one multiply instead of a division by a
// run-time value.  Exact while a * d < 2^32 (the excess of m over 2^32 / d is below one, so the quotient is off by less
// than a / 2^32 < 1 / d); the planes of a plan are held to 2^20 pixels per sample and 2^11 per row for that.  d = 1
// has no 32-bit magic number: a itself, by a select.
inline unsigned plan_magic(int d) { return d <= 1 ? 0u : (unsigned)(0xffffffffu / (unsigned)d + 1u); }
__device__ __forceinline__ int plan_div(int a, unsigned m) {
  const int q = (int)__umulhi((unsigned)a, m);
  return m == 0u ? a : q;
}

// Threads of a workgroup by role: the first PLAN_COMPUTE make the bitmap of a step while PLAN_PIX others write the
// pixel mask of the step before it and the last PLAN_FLG its tile flags, so that none waits for another's
// instruction stream: a step is a few hundred instructions of each kind and nothing else to hide them behind.
constexpr int PLAN_COMPUTE = 640;
constexpr int PLAN_PIX = 192;
constexpr int PLAN_FLG = PLAN_THREADS - PLAN_COMPUTE - PLAN_PIX;

// specialised forms of the footprint (kernel size, stride and "same" padding K / 2 at compile time)
enum { PLAN_KEY_GENERIC = 0, PLAN_KEY_C11, PLAN_KEY_C31, PLAN_KEY_C51, PLAN_KEY_C32, PLAN_KEY_C52, PLAN_KEY_UP, PLAN_KEY_T32, PLAN_KEY_T52 };

// the bitmap of a footprint step: compute thread r of nthr takes words r, r + nthr, ...
template <int FOOT, int K, int S, bool TWO>
__device__ __forceinline__ void plan_foot_all(const PlanStep& s, const uint32_t* bm, uint32_t* out, int r, int nthr) {
  PlanRowAcc<TWO> in;
  in.b1 = bm + s.in1;
  in.b2 = bm + ((TWO && s.in2 >= 0) ? s.in2 : s.in1);
  in.ww = (s.w_in + 31) >> 5;
  in.h = s.h_in;
  const int ho = s.h_out, wo = s.w_out, wwo = (wo + 31) >> 5;
  PlanGeom g;
  g.k = (s.geom >> 8) & 255; g.p = (s.geom >> 24) & 255;
  for (int wd = r; wd < ho * wwo; wd += nthr) {
    const int y = plan_div(wd, s.m_words), j = wd - y * wwo;
    const int left = wo - 32 * j;
    const uint32_t valid = left >= 32 ? 0xffffffffu : ((1u << left) - 1u);
    out[wd] = plan_foot_word<FOOT, K, S, TWO>(g, in, y, j) & valid;
  }
}
template <int FOOT, int K, int S>
__device__ __forceinline__ void plan_foot_any(const PlanStep& s, const uint32_t* bm, uint32_t* out, int r, int nthr) {
  if (s.in2 >= 0) plan_foot_all<FOOT, K, S, true>(s, bm, out, r, nthr);
  else plan_foot_all<FOOT, K, S, false>(s, bm, out, r, nthr);
}

__device__ void plan_compute(const PlanStep& s, const uint32_t* bm, uint32_t* out, int r, int nthr) {
  const int ho = s.h_out, wo = s.w_out, wwo = (wo + 31) >> 5;
  if (s.in1 == PLAN_IN_ALL) {
    for (int wd = r; wd < ho * wwo; wd += nthr) {
      const int j = wd - plan_div(wd, s.m_words) * wwo;
      const int left = wo - 32 * j;
      out[wd] = left >= 32 ? 0xffffffffu : ((1u << left) - 1u);
    }
    return;
  }
  switch (s.key) {       // uniform over the workgroup
    case PLAN_KEY_C11: plan_foot_any<MIE_FOOT_CONV, 1, 1>(s, bm, out, r, nthr); break;
    case PLAN_KEY_C31: plan_foot_any<MIE_FOOT_CONV, 3, 1>(s, bm, out, r, nthr); break;
    case PLAN_KEY_C51: plan_foot_any<MIE_FOOT_CONV, 5, 1>(s, bm, out, r, nthr); break;
    case PLAN_KEY_C32: plan_foot_any<MIE_FOOT_CONV, 3, 2>(s, bm, out, r, nthr); break;
    case PLAN_KEY_C52: plan_foot_any<MIE_FOOT_CONV, 5, 2>(s, bm, out, r, nthr); break;
    case PLAN_KEY_UP: plan_foot_any<MIE_FOOT_UP2X, 1, 1>(s, bm, out, r, nthr); break;
    case PLAN_KEY_T32: plan_foot_any<MIE_FOOT_TCONV, 3, 2>(s, bm, out, r, nthr); break;
    case PLAN_KEY_T52: plan_foot_any<MIE_FOOT_TCONV, 5, 2>(s, bm, out, r, nthr); break;
    default: {
      const int foot = s.geom & 255, ss = (s.geom >> 16) & 255;
      if (foot == MIE_FOOT_TCONV) plan_foot_all<MIE_FOOT_TCONV, 0, 2, true>(s, bm, out, r, nthr);
      else if (ss == 1) plan_foot_all<MIE_FOOT_CONV, 0, 1, true>(s, bm, out, r, nthr);
      else plan_foot_all<MIE_FOOT_CONV, 0, 2, true>(s, bm, out, r, nthr);
    }
  }
}

// What a step leaves in memory, from its bitmap `out`.  The pixel mask, as bytes: this workgroup's slice (share of
// shares), by threads r of nthr.
__device__ void plan_write_pixels(const PlanStep& s, const uint32_t* out, int n, int share, int shares, int r, int nthr) {
  const int ho = s.h_out, wo = s.w_out, wwo = (wo + 31) >> 5;
  const int first = share * nthr + r, stride = shares * nthr;
  uint8_t* pm = s.pixmask + (long long)n * ho * wo;
  if ((wo & 15) == 0) {
    const int per_row = wo >> 4, units = ho * per_row;
    for (int u = first; u < units; u += stride) {
      const int y = plan_div(u, s.m_units), q = u - y * per_row;
      const uint32_t b16 = out[y * wwo + (q >> 1)] >> (16 * (q & 1));
      const uint4 v = make_uint4(plan_bytes(b16 & 15u), plan_bytes((b16 >> 4) & 15u), plan_bytes((b16 >> 8) & 15u),
                                 plan_bytes((b16 >> 12) & 15u));
      *reinterpret_cast<uint4*>(pm + (long long)y * wo + 16 * q) = v;
    }
  } else if ((wo & 3) == 0) {
    const int per_row = wo >> 2, units = ho * per_row;
    for (int u = first; u < units; u += stride) {
      const int y = plan_div(u, s.m_units), q = u - y * per_row;
      const uint32_t nib = (out[y * wwo + (q >> 3)] >> (4 * (q & 7))) & 15u;
      *reinterpret_cast<uint32_t*>(pm + (long long)y * wo + 4 * q) = plan_bytes(nib);
    }
  } else {
    for (int u = first; u < ho * wo; u += stride) {
      const int y = plan_div(u, s.m_units), x = u - y * wo;
      pm[u] = (uint8_t)((out[y * wwo + (x >> 5)] >> (x & 31)) & 1u);
    }
  }
}

// The tile flags: tile (ty, tx) is byte tx % 4 of word tx / 4 in rows 8*ty .. 8*ty+7.  A flag word is written by the one
// thread that owns its tile -- word f of this step's flag area is tile f * shares + share -- from the old value fetched
// at the start.
__device__ void plan_write_flags(const PlanStep& s, const uint32_t* out, const uint32_t* s_old, int n, int share, int shares,
                                 int r, int nthr) {
  const int ho = s.h_out, wo = s.w_out, wwo = (wo + 31) >> 5;
  const int tiles_y = (ho + MIE_TILE - 1) / MIE_TILE, tiles_x = (wo + MIE_TILE - 1) / MIE_TILE;
  const int tpp = tiles_y * tiles_x;
  for (int f = r; f < s.flag_cnt; f += nthr) {
    const int t = f * shares + share;
    if (t >= tpp) break;
    const int ty = plan_div(t, s.m_tiles), tx = t - ty * tiles_x;
    uint32_t any = 0u;
#pragma unroll
    for (int q = 0; q < MIE_TILE; ++q) {
      const int y = ty * MIE_TILE + q;
      any |= out[(y < ho ? y : ho - 1) * wwo + (tx >> 2)] & (y < ho ? 0xffffffffu : 0u);
    }
    s.flags[n * tpp + t] = next_flag(s_old[s.flag_off + f], ((any >> (8 * (tx & 3))) & 0xffu) != 0u);
  }
}

__global__ __launch_bounds__(PLAN_THREADS) void k_plan_bits(PlanArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint32_t plan_lds[];
  // The steps first go from the argument block to LDS in one batch: read where they are used, every step's fields
  // would be a cache miss of their own in a chain where nothing else hides it.
  PlanStep* steps = reinterpret_cast<PlanStep*>(plan_lds);
  uint32_t* bm = plan_lds + PLAN_HEAD;
  const int n = blockIdx.y, tid = threadIdx.x;
  {
    const uint32_t* src = reinterpret_cast<const uint32_t*>(&a.st[0]);
    const int nw = a.n_steps * (int)(sizeof(PlanStep) / 4);
    for (int i = tid; i < nw; i += PLAN_THREADS) plan_lds[i] = src[i];
  }
  __syncthreads();
  // sample blockIdx.y; share blockIdx.x of gridDim.x of everything that is written to memory
  const int share = blockIdx.x, shares = gridDim.x;
  // The tile flags this workgroup owns -- tiles share, share + shares, ... of every set -- hold the previous build's
  // state and are needed when a step is written out.  Asked for step by step, each would be a memory round trip that
  // nothing hides; so all of them are fetched now, in one batch behind which the first mask's loads queue up, into the
  // LDS area in front of the bitmaps (word flag_off + f of a step = tile f * shares + share).
  uint32_t* s_old = bm;
  bm += a.flag_words;
  for (int u = tid; u < a.flag_words; u += PLAN_THREADS) {
    int q = 0;
    for (int i = 1; i < a.n_steps; ++i)
      if (steps[i].flag_off <= u) q = i;            // the last step whose area starts at or below u (areas are in step order)
    const PlanStep& sq = steps[q];
    const int tpp = ((sq.h_out + MIE_TILE - 1) / MIE_TILE) * ((sq.w_out + MIE_TILE - 1) / MIE_TILE);
    const int t = (u - sq.flag_off) * shares + share;
    s_old[u] = (sq.kind == PLAN_STEP_FOOT && t < tpp) ? sq.flags[n * tpp + t] : 0u;
  }
  // role of this wave: 0 = bitmaps, 1 = pixel masks, 2 = tile flags (uniform over a wave: the limits are multiples of 64)
  const int role = tid < PLAN_COMPUTE ? 0 : (tid < PLAN_COMPUTE + PLAN_PIX ? 1 : 2);
  int pending = -1;                                    // the footprint step that is not written out yet
  for (int i = 0; i < a.n_steps; ++i) {
#ifdef MIE_PLAN_PROFILE
    const long long t_step = wall_clock64();
#endif
    const PlanStep s = plan_uni(steps[i]);
    uint32_t* out = bm + s.out;
    const int ho = s.h_out, wo = s.w_out, wwo = (wo + 31) >> 5;
    if (s.kind == PLAN_STEP_LOAD) {
      const uint8_t* src = s.ext + (long long)n * ho * wo;
      for (int wd = tid; wd < ho * wwo; wd += PLAN_THREADS) {
        const int y = plan_div(wd, s.m_words), j = wd - y * wwo;
        const int x0 = 32 * j, nb = (wo - x0 < 32) ? wo - x0 : 32;
        const uint8_t* row = src + (long long)y * wo + x0;
        uint32_t bits = 0u;
        if ((wo & 15) == 0) {           // rows start on 16-byte boundaries and hold whole groups of 16 pixels
          const uint4* r16 = reinterpret_cast<const uint4*>(row);
          const uint4 v0 = r16[0];
          bits = plan_nibble(v0.x) | (plan_nibble(v0.y) << 4) | (plan_nibble(v0.z) << 8) | (plan_nibble(v0.w) << 12);
          if (nb > 16) {
            const uint4 v1 = r16[1];
            bits |= (plan_nibble(v1.x) | (plan_nibble(v1.y) << 4) | (plan_nibble(v1.z) << 8) | (plan_nibble(v1.w) << 12)) << 16;
          }
        } else if ((wo & 3) == 0) {     // 4-byte boundaries
          const uint32_t* r4 = reinterpret_cast<const uint32_t*>(row);
          for (int q = 0; q < (nb >> 2); ++q) bits |= plan_nibble(r4[q]) << (4 * q);
        } else {
          for (int b = 0; b < nb; ++b) bits |= (row[b] != 0 ? 1u : 0u) << b;
        }
        out[wd] = bits;
      }
      __syncthreads();
      continue;
    }
    // The compute waves make this step's bitmap while the others put the step before it into memory.  (They read that
    // step's slot while this step's is written, and the step after this one writes its own one barrier later: the host
    // keeps all three apart -- a slot is handed on one step after its last reader.)
    if (role == 0) {
      plan_compute(s, bm, out, tid, PLAN_COMPUTE);
    } else if (pending >= 0) {
      const PlanStep sp = plan_uni(steps[pending]);
      if (role == 1) plan_write_pixels(sp, bm + sp.out, n, share, shares, tid - PLAN_COMPUTE, PLAN_PIX);
      else plan_write_flags(sp, bm + sp.out, s_old, n, share, shares, tid - PLAN_COMPUTE - PLAN_PIX, PLAN_FLG);
    }
#ifdef MIE_PLAN_PROFILE
    // measurement builds only: ticks of the 100 MHz clock of this step in workgroup (0, 0), first thread of each role
    if (blockIdx.x == 0 && n == 0 && (tid == 0 || tid == PLAN_COMPUTE || tid == PLAN_COMPUTE + PLAN_PIX))
      reinterpret_cast<int32_t*>(a.dbg)[3 * i + role] = (int)(wall_clock64() - t_step);
#endif
    __syncthreads();
    pending = i;
  }
  if (pending >= 0) {       // the last step, by everybody
    const PlanStep sp = plan_uni(steps[pending]);
    plan_write_pixels(sp, bm + sp.out, n, share, shares, tid, PLAN_THREADS);
    plan_write_flags(sp, bm + sp.out, s_old, n, share, shares, tid, PLAN_THREADS);
  }
}

// The lists of every set of a plan: block b is chunk b - first_chunk[i] of the compaction of set i (as
// k_compact_tiles).  The table of first chunks is a few cache lines read in one go; a block then touches only the
// line of its own set.
struct PlanCompactSet {
  int32_t* tiles;
  int32_t* stale;
  int32_t* counts;
  uint32_t* flags;
  int cap, pad_;
};
struct PlanCompactArgs {
  int n_sets, pad_;
  int first_chunk[MIE_PLAN_MAX_STEPS + 2];     // first_chunk[n_sets] = number of blocks
  PlanCompactSet set[MIE_PLAN_MAX_STEPS];
};

__global__ __launch_bounds__(COMPACT_THREADS) void k_plan_compact(PlanCompactArgs a) {
  __shared__ int s_tot[2 * COMPACT_WAVES * COMPACT_ITEMS];
  __shared__ int s_base[2 * COMPACT_WAVES];
  const int b = blockIdx.x;
  int i = 0;
#pragma unroll 1
  for (int q = 1; q < a.n_sets; ++q)
    if (a.first_chunk[q] <= b) i = q;
  const PlanCompactSet& st = a.set[i];
  BuildArgs ba;
  ba.cap = st.cap;
  ba.tiles = st.tiles; ba.stale = st.stale; ba.counts = st.counts; ba.flags = st.flags;
  compact_chunk(ba, b - a.first_chunk[i], a.first_chunk[i + 1] - a.first_chunk[i], s_tot, s_base);
}

// Host side: LDS words of a plane's bitmap.
inline long long plan_words(int h, int w) { return (long long)h * ((w + 31) / 32); }

// First-fit allocator over the bitmap area (word offsets), free blocks kept sorted and coalesced.
struct PlanArena {
  struct Blk { long long off, size; };
  Blk free_[2 * MIE_PLAN_MAX_STEPS + 2];
  int nfree = 0;
  long long top = 0;          // high-water mark
  long long alloc(long long size) {
    for (int i = 0; i < nfree; ++i)
      if (free_[i].size >= size) {
        const long long off = free_[i].off;
        free_[i].off += size;
        free_[i].size -= size;
        if (free_[i].size == 0) {
          for (int j = i; j + 1 < nfree; ++j) free_[j] = free_[j + 1];
          --nfree;
        }
        return off;
      }
    // grow: extend a free block that ends at the top, else start a new one there
    if (nfree > 0 && free_[nfree - 1].off + free_[nfree - 1].size == top) {
      const long long off = free_[nfree - 1].off;
      top = off + size;
      --nfree;
      return off;
    }
    const long long off = top;
    top += size;
    return off;
  }
  void release(long long off, long long size) {
    int i = 0;
    while (i < nfree && free_[i].off < off) ++i;
    for (int j = nfree; j > i; --j) free_[j] = free_[j - 1];
    free_[i] = {off, size};
    ++nfree;
    if (i + 1 < nfree && free_[i].off + free_[i].size == free_[i + 1].off) {
      free_[i].size += free_[i + 1].size;
      for (int j = i + 1; j + 1 < nfree; ++j) free_[j] = free_[j + 1];
      --nfree;
    }
    if (i > 0 && free_[i - 1].off + free_[i - 1].size == free_[i].off) {
      free_[i - 1].size += free_[i].size;
      for (int j = i; j + 1 < nfree; ++j) free_[j] = free_[j + 1];
      --nfree;
    }
  }
};

// LDS a workgroup may use on the current device, and the opt-in for more than 64 KB of it (once per process).
int plan_lds_limit(long long need_bytes, const char* who) {
  static int limit[64];
  static long long opted[64];
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  MIE_REQUIRE(e == hipSuccess && dev >= 0 && dev < 64, MIE_ERR_LAUNCH, "%s: no current device (%s)", who, hipGetErrorString(e));
  if (limit[dev] == 0) {
    int v = 0;
    e = hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev);
    MIE_REQUIRE(e == hipSuccess && v > 0, MIE_ERR_LAUNCH, "%s: cannot read the LDS size of device %d (%s)", who, dev, hipGetErrorString(e));
    limit[dev] = v;
  }
  MIE_REQUIRE(need_bytes <= limit[dev], MIE_ERR_CAPACITY,
              "%s: the masks of this plan need %lld bytes of LDS at once, the device offers %d per workgroup; "
              "build the plan in parts, or with mie_build_mask_tiles", who, need_bytes, limit[dev]);
  if (need_bytes > 65536 && need_bytes > opted[dev]) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(k_plan_bits), hipFuncAttributeMaxDynamicSharedMemorySize, limit[dev]);
    MIE_REQUIRE(e == hipSuccess, MIE_ERR_CAPACITY, "%s: the device refuses %d bytes of dynamic LDS (%s)", who, limit[dev],
                hipGetErrorString(e));
    opted[dev] = limit[dev];
  }
  return MIE_OK;
}

}  // namespace

namespace {
int build_mask_plan(const char* who, const mie_plan_op* ops, int n_ops, int wg_cap, void* stream);
}

extern "C" int mie_build_mask_plan(const mie_plan_op* ops, int n_ops, void* stream) {
  return build_mask_plan("mie_build_mask_plan", ops, n_ops, 0, stream);
}

extern "C" int mie_build_mask_plan_wgs(const mie_plan_op* ops, int n_ops, int max_workgroups, void* stream) {
  const char* who = "mie_build_mask_plan_wgs";
  mie_clear_error();
  MIE_REQUIRE(max_workgroups > 0, MIE_ERR_INVALID_ARG, "%s: max_workgroups %d", who, max_workgroups);
  return build_mask_plan(who, ops, n_ops, max_workgroups, stream);
}

namespace {
int build_mask_plan(const char* who, const mie_plan_op* ops, int n_ops, int wg_cap, void* stream) {
  mie_clear_error();
  MIE_REQUIRE(ops != nullptr && n_ops > 0, MIE_ERR_INVALID_ARG, "%s: no ops", who);
  MIE_REQUIRE(n_ops <= MIE_PLAN_MAX_STEPS, MIE_ERR_CAPACITY, "%s: %d ops, at most %d per call", who, n_ops, MIE_PLAN_MAX_STEPS);
  PlanArgs a;
  memset(&a, 0, sizeof(a));
  a.n = ops[0].out.n;
  // masks in LDS: pointer -> (slot offset, words, step index of the last reader)
  struct Slot { const uint8_t* ptr; long long off, words; int h, w, last, born, rec; };
  // Every allocation of the walk below, with the ops during which it is held (born .. rel, both included): the walk
  // runs twice -- first with a first-fit allocator, which fragments (the short-lived input mask of a UNet leaves a hole
  // that small masks then chop up, and the two full-resolution masks at the end of the chain no longer fit into it);
  // then, if that is tighter, with offsets packed off line from the recorded lifetimes, largest masks first.
  struct AllocRec { long long words, off; int born, rel; };
  AllocRec recs[2 * MIE_PLAN_MAX_STEPS];
  int nrec = 0;
  bool replay = false;
  Slot slots[2 * MIE_PLAN_MAX_STEPS];
  int nslots = 0;
  // which op reads a mask last (by pointer), so that its slot can be handed on afterwards
  auto last_reader = [&](const uint8_t* p, int from) {
    int last = from;
    for (int j = from; j < n_ops; ++j)
      if (ops[j].in_mask == p || ops[j].in_mask2 == p) last = j;
    return last;
  };
  auto find_slot = [&](const uint8_t* p) -> Slot* {
    for (int i = nslots - 1; i >= 0; --i)      // the latest mask at this address
      if (slots[i].ptr == p) return &slots[i];
    return nullptr;
  };
  PlanArena arena;
  long long total_chunks = 0, max_pixels = 0, max_tiles = 0;
  int alloc_no = 0;
  auto slot_alloc = [&](long long words, int born) -> int {      // returns the record index; recs[..].off is the offset
    const int id = alloc_no++;
    if (!replay) {
      recs[id].words = words; recs[id].born = born; recs[id].rel = n_ops;
      recs[id].off = arena.alloc(words);
      nrec = alloc_no;
    }
    return id;
  };
  auto walk = [&]() -> int {
  for (int i = 0; i < n_ops; ++i) {
    const mie_plan_op& op = ops[i];
    int rc = mie_check_tileset(&op.out, who);
    if (rc != MIE_OK) return rc;
    MIE_REQUIRE(op.out.n == a.n, MIE_ERR_INVALID_ARG, "%s: op %d has batch size %d, op 0 has %d", who, i, op.out.n, a.n);
    MIE_REQUIRE(op.h_in > 0 && op.w_in > 0, MIE_ERR_INVALID_ARG, "%s: op %d: input size (%d,%d) must be positive", who, i,
                op.h_in, op.w_in);
    MIE_REQUIRE(op.in_mask != nullptr || op.in_mask2 == nullptr, MIE_ERR_INVALID_ARG, "%s: op %d: in_mask2 given without in_mask", who, i);
    MIE_REQUIRE((long long)a.n * op.h_in * op.w_in < 0x7fffffffLL, MIE_ERR_CAPACITY, "%s: op %d: more than 2^31 input pixels", who, i);
    MIE_REQUIRE(op.w_in <= 2048 && op.out.w <= 2048 && (long long)op.h_in * op.w_in <= (1 << 20) &&
                    (long long)op.out.h * op.out.w <= (1 << 20),
                MIE_ERR_CAPACITY, "%s: op %d: planes of up to 2048 pixels per row and 2^20 pixels per sample (use mie_build_mask_tiles)", who, i);
    const int k = op.k, st = op.stride, pad = op.pad;
    if (op.foot == MIE_FOOT_CONV) {
      MIE_REQUIRE(k >= 1 && k <= 15 && (st == 1 || st == 2) && pad >= 0 && pad < 16, MIE_ERR_UNSUPPORTED,
                  "%s: op %d: conv footprint k=%d stride=%d pad=%d (strides 1 and 2 only)", who, i, k, st, pad);
      const int ho = (op.h_in + 2 * pad - k) / st + 1, wo = (op.w_in + 2 * pad - k) / st + 1;
      MIE_REQUIRE(op.h_in + 2 * pad >= k && op.w_in + 2 * pad >= k && ho == op.out.h && wo == op.out.w, MIE_ERR_INVALID_ARG,
                  "%s: op %d: conv output of (%d,%d) k=%d s=%d p=%d is (%d,%d), tile set is (%d,%d)", who, i, op.h_in, op.w_in, k,
                  st, pad, ho, wo, op.out.h, op.out.w);
    } else if (op.foot == MIE_FOOT_UP2X) {
      MIE_REQUIRE(op.out.h == 2 * op.h_in && op.out.w == 2 * op.w_in, MIE_ERR_INVALID_ARG,
                  "%s: op %d: up2x of (%d,%d) is not (%d,%d)", who, i, op.h_in, op.w_in, op.out.h, op.out.w);
    } else if (op.foot == MIE_FOOT_TCONV) {
      MIE_REQUIRE(k >= 1 && k <= 15 && st == 2 && pad >= 0 && pad < 16, MIE_ERR_UNSUPPORTED,
                  "%s: op %d: tconv footprint k=%d stride=%d pad=%d (stride 2 only)", who, i, k, st, pad);
      const int hmin = (op.h_in - 1) * st - 2 * pad + k, wmin = (op.w_in - 1) * st - 2 * pad + k;
      MIE_REQUIRE(op.out.h >= hmin && op.out.h < hmin + st && op.out.w >= wmin && op.out.w < wmin + st, MIE_ERR_INVALID_ARG,
                  "%s: op %d: tconv output (%d,%d) not in [(%d,%d), +stride)", who, i, op.out.h, op.out.w, hmin, wmin);
    } else {
      MIE_REQUIRE(false, MIE_ERR_UNSUPPORTED, "%s: op %d: unknown footprint %d", who, i, op.foot);
    }
    // (as in mie_build_mask_tiles: only the identity footprint may be built in place)
    const bool identity = op.foot == MIE_FOOT_CONV && k == 1 && st == 1 && pad == 0;
    MIE_REQUIRE(identity || ((const uint8_t*)op.out.pixmask != op.in_mask && (const uint8_t*)op.out.pixmask != op.in_mask2),
                MIE_ERR_INVALID_ARG, "%s: op %d: out.pixmask aliases an input mask (allowed for the 1x1 stride-1 footprint only)", who, i);
    // inputs: a mask an earlier op of this plan wrote is still in LDS; any other is loaded from memory first
    int in_off[2] = {PLAN_IN_NONE, PLAN_IN_NONE};
    const uint8_t* ins[2] = {op.in_mask, op.in_mask2};
    if (op.in_mask == nullptr) in_off[0] = PLAN_IN_ALL;
    for (int q = 0; q < 2 && op.in_mask != nullptr; ++q) {
      if (ins[q] == nullptr) continue;
      Slot* sl = find_slot(ins[q]);
      if (sl == nullptr || sl->last < i) {
        // not in LDS (never was, or its slot has been handed on): load it
        MIE_REQUIRE(a.n_steps < MIE_PLAN_MAX_STEPS && nslots < 2 * MIE_PLAN_MAX_STEPS, MIE_ERR_CAPACITY,
                    "%s: more than %d steps (ops plus masks loaded from memory); build the plan in parts", who, MIE_PLAN_MAX_STEPS);
        Slot ns;
        ns.ptr = ins[q]; ns.h = op.h_in; ns.w = op.w_in; ns.words = plan_words(op.h_in, op.w_in);
        ns.born = i;
        ns.last = last_reader(ins[q], i);
        // (a later op of the plan may overwrite this address: then the mask in LDS is the old one from there on)
        for (int j = i; j < ns.last; ++j)
          if (ops[j].out.pixmask == ins[q]) { ns.last = j; break; }
        ns.rec = slot_alloc(ns.words, i);
        ns.off = recs[ns.rec].off;
        PlanStep& ld = a.st[a.n_steps++];
        ld.kind = PLAN_STEP_LOAD;
        ld.in1 = ld.in2 = PLAN_IN_NONE;
        ld.out = (int)ns.off;
        ld.h_in = ld.h_out = op.h_in; ld.w_in = ld.w_out = op.w_in;
        ld.m_words = plan_magic((op.w_in + 31) / 32);
        ld.ext = ins[q];
        slots[nslots++] = ns;
        sl = &slots[nslots - 1];
      }
      MIE_REQUIRE(sl->h == op.h_in && sl->w == op.w_in, MIE_ERR_INVALID_ARG,
                  "%s: op %d reads a mask of (%d,%d) as (%d,%d)", who, i, sl->h, sl->w, op.h_in, op.w_in);
      in_off[q] = (int)sl->off;
    }
    if (in_off[0] == PLAN_IN_ALL) in_off[1] = PLAN_IN_NONE;
    MIE_REQUIRE(a.n_steps < MIE_PLAN_MAX_STEPS && nslots < 2 * MIE_PLAN_MAX_STEPS, MIE_ERR_CAPACITY,
                "%s: more than %d steps (ops plus masks loaded from memory); build the plan in parts", who, MIE_PLAN_MAX_STEPS);
    // the output's slot: every input of this op is still alive, so it cannot land on one of them
    Slot os;
    os.ptr = op.out.pixmask; os.h = op.out.h; os.w = op.out.w; os.words = plan_words(op.out.h, op.out.w);
    os.last = last_reader(op.out.pixmask, i);
    for (int j = i + 1; j < os.last; ++j)
      if (ops[j].out.pixmask == op.out.pixmask) { os.last = j; break; }      // rewritten before its last reader
    os.born = i;
    // A union (the 1x1 footprint of two masks) is a word-by-word OR: it may overwrite an input that nobody reads after
    // this op -- provided that input is at least two ops old, so that the writer waves of the op before this one, which
    // still read THEIR op's output while this op computes, are not looking at it.  Saves a slot of the plane's size
    // (the full-resolution union at the end of a UNet is what decides whether the chain fits the LDS in one plan).
    os.off = -1;
    if (identity && op.in_mask != nullptr && op.in_mask2 != nullptr) {
      for (int q = 1; q >= 0 && os.off < 0; --q) {
        Slot* sl = find_slot(ins[q]);
        if (sl != nullptr && sl->off == in_off[q] && sl->words == os.words && sl->last == i && sl->born <= i - 2 &&
            ins[q] != (const uint8_t*)op.out.pixmask) {
          os.off = sl->off;
          os.rec = sl->rec;       // the memory is the output's now: one allocation, held on
          sl->words = 0;
          sl->last = -1;
        }
      }
    }
    if (os.off < 0) {
      os.rec = slot_alloc(os.words, i);
      os.off = recs[os.rec].off;
    }
    PlanStep& ft = a.st[a.n_steps++];
    ft.kind = PLAN_STEP_FOOT;
    ft.in1 = in_off[0]; ft.in2 = in_off[1];
    ft.out = (int)os.off;
    ft.h_in = op.h_in; ft.w_in = op.w_in; ft.h_out = op.out.h; ft.w_out = op.out.w;
    ft.geom = op.foot | (k << 8) | (st << 16) | (pad << 24);
    ft.pixmask = op.out.pixmask;
    ft.flags = op.out.flags;
    ft.m_words = plan_magic((op.out.w + 31) / 32);
    ft.m_units = plan_magic(op.out.w % 16 == 0 ? op.out.w / 16 : (op.out.w % 4 == 0 ? op.out.w / 4 : op.out.w));
    ft.m_tiles = plan_magic(mie_div_up(op.out.w, MIE_TILE));
    // the specialised forms have kernel size, stride and the padding k / 2 built in
    ft.key = PLAN_KEY_GENERIC;
    if (op.foot == MIE_FOOT_UP2X) ft.key = PLAN_KEY_UP;
    else if (pad == k / 2) {
      if (op.foot == MIE_FOOT_CONV && st == 1) ft.key = k == 1 ? PLAN_KEY_C11 : k == 3 ? PLAN_KEY_C31 : k == 5 ? PLAN_KEY_C51 : PLAN_KEY_GENERIC;
      if (op.foot == MIE_FOOT_CONV && st == 2) ft.key = k == 3 ? PLAN_KEY_C32 : k == 5 ? PLAN_KEY_C52 : PLAN_KEY_GENERIC;
      if (op.foot == MIE_FOOT_TCONV) ft.key = k == 3 ? PLAN_KEY_T32 : k == 5 ? PLAN_KEY_T52 : PLAN_KEY_GENERIC;
    }
    slots[nslots++] = os;
    // Slots whose last reader was the PREVIOUS op are free from here on: one op late, because the kernel has no
    // barrier between the end of a step (threads still reading its output slot while they write the pixel mask and
    // the flags) and the compute phase of the next step, which writes that step's output slot.  With the release
    // delayed, the slot a step writes was last read at least one whole step -- and its barrier -- earlier.
    for (int q = 0; q < nslots; ++q)
      if (slots[q].last >= 0 && slots[q].last < i && slots[q].words > 0) {
        if (!replay) {
          arena.release(slots[q].off, slots[q].words);
          recs[slots[q].rec].rel = i;
        }
        slots[q].words = 0;
        slots[q].last = -1;
      }
    const int cap = mie_tile_capacity(op.out.n, op.out.h, op.out.w);
    total_chunks += mie_div_up(cap, COMPACT_CHUNK);
    if ((long long)op.out.h * op.out.w > max_pixels) max_pixels = (long long)op.out.h * op.out.w;
    if (cap / op.out.n > max_tiles) max_tiles = cap / op.out.n;
  }
  return MIE_OK;
  };
  int rc = walk();
  if (rc != MIE_OK) return rc;
  {
    // off-line packing: largest first, each at the lowest offset where it meets no allocation whose lifetime overlaps
    int order[2 * MIE_PLAN_MAX_STEPS];
    long long packed[2 * MIE_PLAN_MAX_STEPS];
    for (int i = 0; i < nrec; ++i) order[i] = i;
    for (int i = 1; i < nrec; ++i)
      for (int j = i; j > 0 && (recs[order[j]].words > recs[order[j - 1]].words ||
                                (recs[order[j]].words == recs[order[j - 1]].words && recs[order[j]].born < recs[order[j - 1]].born)); --j) {
        const int t = order[j]; order[j] = order[j - 1]; order[j - 1] = t;
      }
    long long top = 0;
    for (int oi = 0; oi < nrec; ++oi) {
      const AllocRec& r = recs[order[oi]];
      long long off = 0;
      for (bool moved = true; moved;) {
        moved = false;
        for (int oj = 0; oj < oi; ++oj) {
          const AllocRec& q = recs[order[oj]];
          const long long qo = packed[order[oj]];
          if (r.born <= q.rel && q.born <= r.rel && off < qo + q.words && qo < off + r.words) {
            off = qo + q.words;
            moved = true;
          }
        }
      }
      packed[order[oi]] = off;
      if (off + r.words > top) top = off + r.words;
    }
    if (top < arena.top) {
      for (int i = 0; i < nrec; ++i) recs[i].off = packed[i];
      arena.top = top;
      replay = true;
      memset(&a, 0, sizeof(a));
      a.n = ops[0].out.n;
      nslots = 0; alloc_no = 0; total_chunks = 0; max_pixels = 0; max_tiles = 0;
      rc = walk();
      if (rc != MIE_OK) return rc;
    }
  }
  // workgroups per sample: a slice of the largest plane's stores each, and never more than one tile flag per thread
  long long shares = (max_pixels + PLAN_PIXELS_PER_SHARE - 1) / PLAN_PIXELS_PER_SHARE;
  // Every workgroup walks the whole chain of its sample (and loads every mask that comes from memory): with a batch of
  // samples there are workgroups enough without many per sample, and more than one per CU would only queue (a
  // workgroup of a large plane takes most of a CU's LDS).
  static const int max_wgs = [] { const char* e = getenv("MIE_PLAN_WGS"); return e ? atoi(e) : 256; }();      // tuning knob
  const int wgs = (wg_cap > 0 && wg_cap < max_wgs) ? wg_cap : max_wgs;     // a caller's cap: the plan runs beside other kernels
  if (shares * a.n > wgs) shares = wgs / a.n > 0 ? wgs / a.n : 1;
  if (shares * PLAN_THREADS < max_tiles) shares = (max_tiles + PLAN_THREADS - 1) / PLAN_THREADS;
  // the flag area of a workgroup: per set, the tiles it owns (every shares-th one)
  for (int i = 0; i < a.n_steps; ++i) {
    PlanStep& stp = a.st[i];
    stp.flag_off = a.flag_words;
    stp.flag_cnt = 0;
    if (stp.kind != PLAN_STEP_FOOT) continue;
    const long long tpp = (long long)mie_div_up(stp.h_out, MIE_TILE) * mie_div_up(stp.w_out, MIE_TILE);
    stp.flag_cnt = (int)((tpp + shares - 1) / shares);
    a.flag_words += stp.flag_cnt;
  }
  MIE_REQUIRE(shares <= PLAN_MAX_SHARES, MIE_ERR_CAPACITY,
              "%s: a plane of %lld pixels (%lld tiles) per sample is beyond the plan's %d workgroups per sample; use "
              "mie_build_mask_tiles", who, max_pixels, max_tiles, PLAN_MAX_SHARES);
  const long long lds_bytes = (PLAN_HEAD + a.flag_words + arena.top) * 4;
  rc = plan_lds_limit(lds_bytes, who);
  if (rc != MIE_OK) return rc;
#ifdef MIE_PLAN_PROFILE
  a.dbg = reinterpret_cast<int*>(ops[n_ops - 1].out.stale) + (mie_tile_capacity(a.n, ops[n_ops - 1].out.h, ops[n_ops - 1].out.w) - 3 * MIE_PLAN_MAX_STEPS);
#endif
  hipLaunchKernelGGL(k_plan_bits, dim3((unsigned)shares, (unsigned)a.n), dim3(PLAN_THREADS), (size_t)lds_bytes,
                     (hipStream_t)stream, a);
  rc = mie_check_launch(who);
  if (rc != MIE_OK) return rc;
  PlanCompactArgs c;
  memset(&c, 0, sizeof(c));
  for (int i = 0; i < n_ops; ++i) {
    const mie_tileset& ts = ops[i].out;
    PlanCompactSet& st = c.set[c.n_sets];
    st.tiles = ts.tiles; st.stale = ts.stale; st.counts = ts.counts; st.flags = ts.flags;
    st.cap = mie_tile_capacity(ts.n, ts.h, ts.w);
    c.first_chunk[c.n_sets + 1] = c.first_chunk[c.n_sets] + mie_div_up(st.cap, COMPACT_CHUNK);
    ++c.n_sets;
  }
  hipLaunchKernelGGL(k_plan_compact, dim3((unsigned)total_chunks), dim3(COMPACT_THREADS), 0, (hipStream_t)stream, c);
  return mie_check_launch(who);
}
}  // namespace
