// Masked conv on the fp32 matrix cores (v_mfma_f32_32x32x2_f32), gfx950.
//
// Work decomposition.  One 256-thread workgroup (4 waves) computes one active
// 8x8 output tile (M = 64 pixels) x CO_BLK output channels as an implicit GEMM
// over k = (input channel, tap):
//   * A (pixels x k): the input tile plus halo is staged in LDS, CC input
//     channels at a time, by all 256 threads with 16-byte loads of the NHWC
//     rows; pixels whose mask byte is 0 (or that lie outside the image) are
//     zero-filled without touching HBM.  Staging is double buffered: the
//     global loads of chunk c+1 are in flight while chunk c is multiplied.
//   * B (k x channels): filter rows filt[ci][ky][kx][co..co+31] are read
//     straight from L2 into registers (each value is used by exactly one wave
//     of the workgroup), one unit ahead of the MFMAs that consume them.
//   * The 4 waves split the workgroup's work WN ways over output channels and
//     WK = 4/WN ways over k (units = tap x 8-channel sub-chunk, round robin).
//     Layers with few tiles (33x44 bottleneck: 30 tiles) take WN=1, WK=4 so
//     that tiles x Cout/32 workgroups of 4 busy waves fill the chip; wide
//     layers take WN=4.  K-split partial sums meet in LDS and are added in a
//     fixed order (bit-reproducible).
// A lane's operand layout: lanes 0-31 = the 32 pixels of an M block, the lane
// half selects 4 of the 8 channels of a sub-chunk, read as ONE ds_read_b128
// that feeds 4 k-steps (k-step j pairs channel j of the low half with channel
// 4+j of the high half; the B operand is loaded with the same pairing).  The
// LDS row stride CC+4 floats keeps the 16-byte reads of 8 neighbouring pixels
// on disjoint banks for stride 1 and 2.
#include "mie_conv.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

template <int K, int S, int WN, int NB>
__global__ __launch_bounds__(256) void k_conv_mfma(ConvArgs a) {
  constexpr int WK = 4 / WN;
  constexpr int IT = 7 * S + K;                              // input tile edge incl. halo
  constexpr int CC = (K == 7) ? 8 : (S == 2 ? 16 : 32);      // channels per LDS stage
  constexpr int LS = CC + 4;                                 // LDS floats per staged pixel
  constexpr int NPIX = IT * IT;
  constexpr int Q4 = CC / 4;                                 // float4 slots per pixel
  constexpr int NSLOT = NPIX * Q4;
  constexpr int NLD = (NSLOT + 255) / 256;                   // staging loads per thread
  constexpr int STAGE = NPIX * LS;                           // floats per staging buffer
  constexpr int NQ = CC / 8;                                 // 8-channel sub-chunks per stage
  constexpr int UNITS = K * K * NQ;                          // (tap, sub-chunk) units per stage
  constexpr int CO_BLK = 32 * NB * WN;
  constexpr int RED = (WK > 1) ? WK * 64 * CO_BLK : 0;
  constexpr int SMEM = (2 * STAGE > RED) ? 2 * STAGE : RED;
  static_assert(SMEM * 4 <= 65536, "LDS budget");
  __shared__ __attribute__((aligned(16))) float smem[SMEM];

  int n, y0, x0;
  const int tk = mie_pick_tile(a.ts, blockIdx.x, n, y0, x0);
  if (tk == 0) return;
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int wn = wave % WN, wk = wave / WN;
  const int co0 = blockIdx.y * CO_BLK;
  const int hout = a.ts.h, wout = a.ts.w;

  if (tk == 2) {  // stale tile: zero this workgroup's channel slab
    for (int idx = tid; idx < 64 * CO_BLK; idx += 256) {
      const int p = idx / CO_BLK, col = idx - p * CO_BLK;
      const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
      if (oy < hout && ox < wout)
        a.out[(((long long)n * hout + oy) * wout + ox) * a.cout + co0 + col] = 0.f;
    }
    return;
  }

  v16f acc[2][NB];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mb][nb][r] = 0.f;

  // ---- per-thread staging plan: which pixels / float4 slots this thread copies -------------
  const int iy0 = y0 * S - a.pad, ix0 = x0 * S - a.pad;
  int st_po[NLD];       // linear input pixel index, -1 = outside the image / beyond the tile
  int st_lds[NLD];      // LDS float offset of the slot
  int st_c4[NLD];       // channel offset of the slot inside the chunk
  unsigned ok1 = 0u, ok2 = 0u;   // slot readable from x / x2 (pixel mask set)
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int slot = tid + 256 * i;
    const int pix = slot / Q4, q4 = slot - pix * Q4;
    st_lds[i] = pix * LS + 4 * q4;
    st_c4[i] = 4 * q4;
    st_po[i] = -1;
    if (slot < NSLOT) {
      const int iy = iy0 + pix / IT, ix = ix0 + pix % IT;
      if (iy >= 0 && iy < a.h_in && ix >= 0 && ix < a.w_in) {
        const int po = (n * a.h_in + iy) * a.w_in + ix;
        st_po[i] = po;
        if (a.xm == nullptr || a.xm[po]) ok1 |= 1u << i;
        if (a.x2 != nullptr && (a.x2m == nullptr || a.x2m[po])) ok2 |= 1u << i;
      }
    }
  }
  const int nch1 = (a.c1 + CC - 1) / CC;
  const int nch = nch1 + ((a.x2 != nullptr) ? (a.c2 + CC - 1) / CC : 0);

  float4 st_reg[NLD];
  auto stage_load = [&](int c) {
    const bool second = c >= nch1;
    const float* xin = second ? a.x2 : a.x;
    const int cs = second ? a.c2 : a.c1;
    const int ci0 = (second ? c - nch1 : c) * CC;
    const unsigned ok = second ? ok2 : ok1;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (((ok >> i) & 1u) && ci0 + st_c4[i] < cs)
        v = *reinterpret_cast<const float4*>(xin + (long long)st_po[i] * cs + ci0 + st_c4[i]);
      st_reg[i] = v;
    }
  };
  auto stage_store = [&](int buf) {
    float* dst = smem + buf * STAGE;
#pragma unroll
    for (int i = 0; i < NLD; ++i)
      if (tid + 256 * i < NSLOT) *reinterpret_cast<float4*>(dst + st_lds[i]) = st_reg[i];
  };

  // ---- B operand: filter rows for unit u of chunk c ------------------------------------------------
  const int cob = co0 + wn * (32 * NB) + l32;
  auto unit_valid = [&](int c, int u) {
    const bool second = c >= nch1;
    const int cs = second ? a.c2 : a.c1;
    const int ci0 = (second ? c - nch1 : c) * CC;
    return ci0 + 8 * (u % NQ) < cs;
  };
  auto load_b = [&](int c, int u, float (&bv)[NB][4]) {
    const bool second = c >= nch1;
    const int ci0 = (second ? c - nch1 : c) * CC;
    const int fb = second ? a.c1 : 0;
    const int tap = u / NQ, q = u - tap * NQ;
    const float* wp = a.filt + ((long long)(fb + ci0 + 8 * q + 4 * half) * (K * K) + tap) * a.cout + cob;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) bv[nb][j] = wp[(long long)j * (K * K) * a.cout + nb * 32];
  };

  // LDS pixel index of this lane's output pixel in M block mb at tap (0,0)
  int pbase[2];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {
    const int p = mb * 32 + l32;
    pbase[mb] = ((p >> 3) * S) * IT + (p & 7) * S;
  }

  float bcur[NB][4], bnext[NB][4];
  stage_load(0);
  if (wk < UNITS && unit_valid(0, wk)) load_b(0, wk, bcur);
  stage_store(0);
  __syncthreads();

  for (int c = 0; c < nch; ++c) {
    const bool more = c + 1 < nch;
    if (more) stage_load(c + 1);
    const float* sin = smem + (c & 1) * STAGE;
#pragma unroll 1
    for (int u = wk; u < UNITS; u += WK) {
      // prefetch B of the next unit (possibly the first unit of the next chunk)
      int c2 = c, u2 = u + WK;
      if (u2 >= UNITS) { c2 = c + 1; u2 = wk; }
      if (c2 < nch && u2 < UNITS && unit_valid(c2, u2)) load_b(c2, u2, bnext);
      if (unit_valid(c, u)) {
        const int tap = u / NQ, q = u - tap * NQ;
        const int ky = tap / K, kx = tap - ky * K;
        float4 av[2];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
          av[mb] = *reinterpret_cast<const float4*>(
              &sin[(pbase[mb] + ky * IT + kx) * LS + 8 * q + 4 * half]);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
              acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32((&av[mb].x)[j], bcur[nb][j],
                                                                 acc[mb][nb], 0, 0, 0);
      }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int j = 0; j < 4; ++j) bcur[nb][j] = bnext[nb][j];
    }
    if (more) stage_store((c + 1) & 1);
    __syncthreads();
  }

  // ---- epilogue -----------------------------------------------------------------------------------
  // acc[mb][nb][r] of this lane is output pixel p = 32*mb + 8*(r/4) + 4*half + r%4,
  // channel column wn*32*NB + 32*nb + lane%32 of the workgroup's slab.
  if (WK == 1) {
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int p = mb * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
        const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
        if (oy >= hout || ox >= wout) continue;
        const long long ob = (((long long)n * hout + oy) * wout + ox) * a.cout + cob;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) conv_store(a, ob + nb * 32, acc[mb][nb][r]);
      }
  } else {
    // the trailing barrier of the main loop has retired every read of the staging buffers
    float* red = smem + wk * (64 * CO_BLK);
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int p = mb * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
          red[p * CO_BLK + wn * (32 * NB) + nb * 32 + l32] = acc[mb][nb][r];
      }
    __syncthreads();
    for (int idx = tid; idx < 64 * CO_BLK; idx += 256) {
      const int p = idx / CO_BLK, col = idx - p * CO_BLK;
      const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
      if (oy >= hout || ox >= wout) continue;
      float s = smem[idx];
#pragma unroll
      for (int k2 = 1; k2 < WK; ++k2) s += smem[k2 * (64 * CO_BLK) + idx];
      conv_store(a, (((long long)n * hout + oy) * wout + ox) * a.cout + co0 + col, s);
    }
  }
}

template <int K, int S>
void launch_ks(const ConvArgs& a, unsigned cap, hipStream_t st) {
  // Pick the widest channel slab that still gives the chip enough workgroups
  // (256 CUs; aim for >= 2 workgroups per CU when every tile is active).
  const long long want = 512;
  if (a.cout % 256 == 0 && (long long)cap * (a.cout / 256) >= want)
    hipLaunchKernelGGL((k_conv_mfma<K, S, 4, 2>), dim3(cap, a.cout / 256), dim3(256), 0, st, a);
  else if (a.cout % 128 == 0 && (long long)cap * (a.cout / 128) >= want)
    hipLaunchKernelGGL((k_conv_mfma<K, S, 4, 1>), dim3(cap, a.cout / 128), dim3(256), 0, st, a);
  else if (a.cout % 64 == 0 && (long long)cap * (a.cout / 64) >= want)
    hipLaunchKernelGGL((k_conv_mfma<K, S, 2, 1>), dim3(cap, a.cout / 64), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL((k_conv_mfma<K, S, 1, 1>), dim3(cap, a.cout / 32), dim3(256), 0, st, a);
}

}  // namespace

void mie_launch_conv_mfma(const ConvArgs& a, int k, int s, unsigned cap, hipStream_t st) {
  switch (k * 10 + s) {
    case 11: launch_ks<1, 1>(a, cap, st); break;
    case 12: launch_ks<1, 2>(a, cap, st); break;
    case 31: launch_ks<3, 1>(a, cap, st); break;
    case 32: launch_ks<3, 2>(a, cap, st); break;
    case 51: launch_ks<5, 1>(a, cap, st); break;
    case 52: launch_ks<5, 2>(a, cap, st); break;
    case 71: launch_ks<7, 1>(a, cap, st); break;
    case 72: launch_ks<7, 2>(a, cap, st); break;
    default: break;  // unreachable: the caller validated k and s
  }
}
