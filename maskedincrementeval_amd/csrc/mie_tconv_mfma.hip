// Stride-2 transposed conv of a delta on the matrix cores (gfx950): kernel size K in {3, 5}, padding
// K/2, output exactly twice the input (output_padding 1) -- the decoder layer of the flow and depth
// networks (incr_modules/e2depth_incr.py:243-282).
//
// Sub-pixel decomposition.  Output row 2i + py receives input row i + dy through tap ky iff
// py == (ky - pad) mod 2, with dy = (py + pad - ky) / 2; the same holds for columns.  The four output
// phases (py, px) are therefore four ordinary stride-1 contractions over disjoint tap subsets of the
// same staged input: for K = 3 phase (0,0) has 1 tap, (0,1) and (1,0) two, (1,1) four -- 9 taps for
// 4 output pixels, where the zero-insertion form would multiply 36.  One workgroup takes an 8x8 block
// of INPUT positions (a 16x16 block of output pixels): M = 64 positions per phase, four accumulator sets,
// the input block plus halo staged once per channel chunk exactly as in the conv kernel
// (mie_conv_mfma_impl.h: same LDS layout, operand pairing, filter ring and k-split), each tap's MFMAs
// going to the accumulators of its phase.  No multiplication is wasted on inserted zeros.
//
// Tile sets.  `a.ts` is the output tile set (8x8 output tiles, MIE_FOOT_TCONV); the workgroups walk `pts`,
// the tile set of the 16x16 output blocks at input resolution (built from the output pixel mask with a 2x2
// stride-2 OR): a block is live when any of its four output tiles is.  A live block writes all its 256
// pixels (zeros where no input reaches), a stale block is zeroed, which covers every stale output tile.
// On planes of very few blocks the chunks are split over gridDim.z workgroups that write partial sums to the
// workspace, and k_conv_split_finish (walking the OUTPUT tile set) adds them and runs the epilogue.
#include "mie_conv_mfma_impl.h"
#include <type_traits>

namespace {

__host__ __device__ constexpr int tc_phase(int k, int pad) { return (((k - pad) % 2) + 2) % 2; }
__host__ __device__ constexpr int tc_shift(int k, int pad) { return (tc_phase(k, pad) + pad - k) / 2; }   // numerator is even

// X3 (fp32 deltas): the three-term bf16 form of k_conv_mfma -- staged values and weights as hi + mid + lo in bf16, six
// v_mfma_f32_32x32x16_bf16 products per multiply, fp32 accuracy; chunks of 64 channels (four units per tap, so that the
// k-split stays over whole sub-chunks and every tap's phase is known at compile time), three bf16 planes in LDS,
// single-buffered.  With the accumulators of four phases it needs 140-176 registers beside them: one workgroup per CU
// (forcing two makes it spill and costs 1 % of the EVFlowNet frame; as it is the form gains 1-2 % there).
template <typename T, int K, int WN, bool SPLIT, bool X3 = false>
__global__ __launch_bounds__(256) void k_tconv_mfma(ConvArgsT<T> a, TileSetDev pts) {
  static_assert(!X3 || sizeof(T) == 4, "X3: fp32 deltas");
  using TL = std::conditional_t<X3, mie_bf16, T>;            // element type in LDS and on the matrix cores
  constexpr int PL = X3 ? 3 : 1;                             // operand planes (terms per value)
  constexpr int GPS = X3 ? 2 : 1;                            // 16-byte global loads per staging slot
  constexpr int PAD = K / 2;
  constexpr int LO = (K == 5) ? 1 : 0;                       // halo above / left of the block (shifts reach -LO .. +1)
  constexpr int NBUF = X3 ? 1 : stage_buffers(1, (int)sizeof(T));
  constexpr int EPS = 16 / (int)sizeof(TL);
  constexpr int SUB = 2 * EPS;
  constexpr int WK = 4 / WN;
  constexpr int IT = 8 + LO + 1;
  constexpr int CC = X3 ? 64 : stage_channels(K, 1) * (4 / (int)sizeof(T));
  constexpr int LS = CC + EPS;
  constexpr int NPIX = IT * IT;
  constexpr int Q4 = CC / EPS;
  constexpr int NSLOT = NPIX * Q4;
  constexpr int NLD = (NSLOT + 255) / 256;
  constexpr int RP = row_pitch_dw(IT, LS * (int)sizeof(TL) / 4, 1) * 4 / (int)sizeof(TL);
  constexpr int STAGE = IT * RP;                             // elements per plane of a staging buffer
  constexpr int NQ = CC / SUB;
  static_assert(NQ % WK == 0, "the k-split is over whole sub-chunks");
  constexpr int NQW = NQ / WK;
  constexpr int UPC = K * K * NQW;
  constexpr int RING = (X3 && ring_size(UPC) > 6) ? ring_size(UPC, 3) : ring_size(UPC);
  constexpr int PD = RING - 1;
  constexpr int CO_BLK = 32 * WN;
  constexpr int RED = WK * 64 * CO_BLK;                      // the accumulators of one phase, parked for the epilogue
  constexpr int STAGE_F = NBUF * PL * STAGE * (int)sizeof(TL) / 4;
  constexpr int SMEM = STAGE_F > RED ? STAGE_F : RED;
  static_assert(SMEM * 4 <= 65536, "LDS budget");
  static_assert(!SPLIT || WN == 1, "the split form is the 32-channel slab kernel");
  __shared__ __attribute__((aligned(16))) float smem[SMEM];
  TL* const sbuf = reinterpret_cast<TL*>(smem);

  int n, y0, x0;                                             // block origin in INPUT coordinates
  const int tk = mie_pick_tile(pts, blockIdx.x + conv_args_entry_zero(a), n, y0, x0);
  if (tk == 0) return;
  const int by = blockIdx.y, bz = SPLIT ? (int)blockIdx.z : 0;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int wn = wave % WN, wk = wave / WN;
  const int co0 = by * CO_BLK;
  const int hout = 2 * a.h_in, wout = 2 * a.w_in;
  const int cout = a.cout;

  if (tk == 2) {                                             // stale block: zero this workgroup's slab of its 16x16 pixels
    if (SPLIT) return;                                       // (the finish kernel zeroes the stale output tiles)
    for (int idx = tid; idx < 64 * CO_BLK; idx += 256) {      // groups of four channels
      const int p = idx / (CO_BLK / 4), col = 4 * (idx - p * (CO_BLK / 4));
      const int oy = 2 * y0 + (p >> 4), ox = 2 * x0 + (p & 15);
      if (oy < hout && ox < wout)
        mie_st4(a.out, (((long long)n * hout + oy) * wout + ox) * cout + co0 + col, make_float4(0.f, 0.f, 0.f, 0.f));
    }
    return;
  }

  v16f acc[4][2];
#pragma unroll
  for (int ph = 0; ph < 4; ++ph)
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ph][mb][r] = 0.f;

  // ---- staging plan (as in k_conv_mfma, stride 1) ------------------------------------------------------
  const int iy0 = y0 - LO, ix0 = x0 - LO;
  int st_po[NLD], st_lds[NLD], st_c4[NLD];
  unsigned ok1 = 0u, ok2 = 0u;
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int slot = tid + 256 * i;
    const int pix = slot / Q4, q4 = slot - pix * Q4;
    const int lrow = pix / IT;
    st_lds[i] = lrow * RP + (pix - lrow * IT) * LS + EPS * q4;
    st_c4[i] = EPS * q4;
    st_po[i] = 0;
    if (slot < NSLOT) {
      const int iy = iy0 + lrow, ix = ix0 + (pix - lrow * IT);
      if (iy >= 0 && iy < a.h_in && ix >= 0 && ix < a.w_in) {
        const int po = (n * a.h_in + iy) * a.w_in + ix;
        st_po[i] = po;
        if (a.xm == nullptr || a.xm[po]) ok1 |= 1u << i;
        if (a.x2 != nullptr && (a.x2m == nullptr || a.x2m[po])) ok2 |= 1u << i;
      }
    }
  }
  const int nch1 = a.c1 / CC;
  const int nch = nch1 + (a.x2 != nullptr ? a.c2 / CC : 0);

  float4 st_reg[NLD][GPS];
  auto stage_load = [&](int c) {
    const bool second = c >= nch1;
    const T* xin = second ? a.x2 : a.x;
    const int cs = second ? a.c2 : a.c1;
    const int ci0 = (second ? c - nch1 : c) * CC;
    const unsigned ok = second ? ok2 : ok1;
    const T* dummy = a.filt_mc;          // masked lanes read one cache-resident address: loads stay unconditional
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const bool okb = (ok >> i) & 1u;
      const T* p = xin + (long long)st_po[i] * cs + ci0 + st_c4[i];
      p = okb ? p : dummy;
#pragma unroll
      for (int g = 0; g < GPS; ++g) {
        float4 v = *reinterpret_cast<const float4*>(p + 4 * g);
        v.x = okb ? v.x : 0.f; v.y = okb ? v.y : 0.f; v.z = okb ? v.z : 0.f; v.w = okb ? v.w : 0.f;
        st_reg[i][g] = v;
      }
    }
  };
  auto stage_store = [&](int buf) {
    TL* dst = sbuf + buf * (PL * STAGE);
#pragma unroll
    for (int i = 0; i < NLD; ++i)
      if (tid + 256 * i < NSLOT) {
        if constexpr (X3) {
          const float f[8] = {st_reg[i][0].x, st_reg[i][0].y, st_reg[i][0].z, st_reg[i][0].w,
                              st_reg[i][1].x, st_reg[i][1].y, st_reg[i][1].z, st_reg[i][1].w};
          float4 pl[3];
          split3(f, pl);
#pragma unroll
          for (int q = 0; q < 3; ++q) *reinterpret_cast<float4*>(dst + q * STAGE + st_lds[i]) = pl[q];
        } else {
          *reinterpret_cast<float4*>(dst + st_lds[i]) = st_reg[i][0];
        }
      }
  };

  // ---- operand addressing --------------------------------------------------------------------------------
  const int q0w = wk * NQW;
  const int cob0 = co0 + wn * 32;
  const int b_lane = (half * cout + l32) * EPS;
  int a_lane[2];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {
    const int p = mb * 32 + l32;
    a_lane[mb] = (p >> 3) * RP + (p & 7) * LS + SUB * q0w + EPS * half;
  }
  auto chunk_b = [&](int c) -> const TL* {
    const bool second = c >= nch1;
    const int ci0 = (second ? c - nch1 : c) * CC;
    const int fb = second ? a.c1 : 0;
    return reinterpret_cast<const TL*>(a.filt_mc) + ((long long)((fb + ci0) / SUB + q0w) * (K * K) * (PL * 2) * cout + cob0) * EPS;
  };
  float4 bring[RING][PL];
  auto load_b = [&](const TL* ub, int unit, float4 (&bv)[PL]) {
    const int tap = unit / NQW, qi = unit % NQW;
#pragma unroll
    for (int q = 0; q < PL; ++q)
      bv[q] = *reinterpret_cast<const float4*>(ub + ((long long)(((qi * (K * K) + tap) * PL + q) * 2) * cout) * EPS + b_lane);
  };

  const int c_lo = SPLIT ? bz * nch / (int)gridDim.z : 0;
  const int c_hi = SPLIT ? (bz + 1) * nch / (int)gridDim.z : nch;
  const TL* ub_cur = chunk_b(c_lo);
  const TL* ub_next = ub_cur;
  stage_load(c_lo);
#pragma unroll
  for (int i = 0; i < (PD > 0 ? PD : 1); ++i) load_b(ub_cur, i, bring[i % RING]);
  stage_store(0);
  __syncthreads();

  for (int c = c_lo; c < c_hi; ++c) {
    const bool more = c + 1 < c_hi;
    const int cn = more ? c + 1 : c;
    ub_next = chunk_b(cn);
    stage_load(cn);
    const TL* sin = sbuf + ((c - c_lo) % NBUF) * (PL * STAGE);
    float4 av[2][2][PL];
    auto load_a = [&](int unit, float4 (&dst)[2][PL]) {
      const int tap = unit / NQW, qi = unit % NQW;
      const int ky = tap / K, kx = tap - ky * K;
      const int dy = tc_shift(ky, PAD) + LO, dx = tc_shift(kx, PAD) + LO;
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int q = 0; q < PL; ++q)
          dst[mb][q] = *reinterpret_cast<const float4*>(&sin[q * STAGE + a_lane[mb] + dy * RP + dx * LS + SUB * qi]);
    };
    load_a(0, av[0]);
#pragma unroll
    for (int i = 0; i < UPC; ++i) {
      if (PD > 0) {
        const int ip = i + PD;
        if (ip < UPC) load_b(ub_cur, ip, bring[ip % RING]);
        else load_b(ub_next, ip - UPC, bring[ip % RING]);
      }
      if (i + 1 < UPC) load_a(i + 1, av[(i + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
      {
        const int tap = i / NQW;
        const int ky = tap / K, kx = tap - ky * K;
        const int ph = tc_phase(ky, PAD) * 2 + tc_phase(kx, PAD);      // compile-time after unrolling
        if constexpr (X3) {
          // the six significant term products of the unit, the two pixel blocks interleaved (smallest terms first)
          const auto& A = av[i & 1];
          const auto& B = bring[i % RING];
          mma_unit(acc[ph][0], A[0][2], B[0], mie_bf16()); mma_unit(acc[ph][1], A[1][2], B[0], mie_bf16());
          mma_unit(acc[ph][0], A[0][1], B[1], mie_bf16()); mma_unit(acc[ph][1], A[1][1], B[1], mie_bf16());
          mma_unit(acc[ph][0], A[0][0], B[2], mie_bf16()); mma_unit(acc[ph][1], A[1][0], B[2], mie_bf16());
          mma_unit(acc[ph][0], A[0][1], B[0], mie_bf16()); mma_unit(acc[ph][1], A[1][1], B[0], mie_bf16());
          mma_unit(acc[ph][0], A[0][0], B[1], mie_bf16()); mma_unit(acc[ph][1], A[1][0], B[1], mie_bf16());
          mma_unit(acc[ph][0], A[0][0], B[0], mie_bf16()); mma_unit(acc[ph][1], A[1][0], B[0], mie_bf16());
        } else {
#pragma unroll
          for (int mb = 0; mb < 2; ++mb) mma_unit(acc[ph][mb], av[i & 1][mb][0], bring[i % RING][0], T());
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if (PD == 0) load_b(ub_next, 0, bring[0]);
    }
    if (NBUF == 1) __syncthreads();
    if (more) stage_store((c - c_lo + 1) % NBUF);
    __syncthreads();
    ub_cur = ub_next;
  }

  // ---- epilogue, one phase at a time -----------------------------------------------------------------------
  // acc[ph][mb][r] of this lane: input position p = 32*mb + 8*(r/4) + 4*half + r%4 of the block, i.e. output
  // pixel (2*(y0 + p/8) + py, 2*(x0 + p%8) + px), channel column wn*32 + lane%32 of the slab.
  // (a generic lambda called once per phase: the accumulator set is picked at compile time)
  auto epilogue = [&](auto PH) {
    constexpr int ph = decltype(PH)::value;
    constexpr int py = ph >> 1, px = ph & 1;
    // every wave parks the phase's accumulators in LDS; a thread then owns groups of four adjacent output channels
    // of a pixel (16-byte reads of the k-split partial sums, 16-byte reservoir accesses, 16- / 8-byte delta accesses)
    constexpr int QPP = CO_BLK / 4;
    constexpr int PER = 64 * QPP / 256;
    float* red = smem + wk * (64 * CO_BLK);
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int p = mb * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
        red[p * CO_BLK + wn * 32 + l32] = acc[ph][mb][r];
      }
    __syncthreads();
    long long off[PER];
    int co[PER];
    bool ok[PER];
    float4 v[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = tid + 256 * i;
      const int p = idx / QPP, col = 4 * (idx - p * QPP);
      const int iy = y0 + (p >> 3), ix = x0 + (p & 7);
      ok[i] = iy < a.h_in && ix < a.w_in;
      off[i] = (((long long)n * hout + 2 * iy + py) * wout + 2 * ix + px) * cout + co0 + col;
      co[i] = co0 + col;
      float4 sum = *reinterpret_cast<const float4*>(&smem[4 * idx]);
#pragma unroll
      for (int k2 = 1; k2 < WK; ++k2) {
        const float4 part = *reinterpret_cast<const float4*>(&smem[k2 * (64 * CO_BLK) + 4 * idx]);
        sum.x += part.x; sum.y += part.y; sum.z += part.z; sum.w += part.w;
      }
      v[i] = sum;
    }
    if constexpr (SPLIT) {
      float* plane = a.ws + (long long)bz * a.ws_plane;
#pragma unroll
      for (int i = 0; i < PER; ++i)
        if (ok[i]) *reinterpret_cast<float4*>(plane + off[i]) = v[i];
    } else {
      float4 r0[PER], add[PER];
      conv_epilogue_load4<T, PER>(a, off, ok, r0, add);
      conv_epilogue_store4<T, PER>(a, off, co, ok, v, r0, add);
    }
    __syncthreads();                   // the next phase overwrites the parked accumulators
  };
  epilogue(std::integral_constant<int, 0>{});
  epilogue(std::integral_constant<int, 1>{});
  epilogue(std::integral_constant<int, 2>{});
  epilogue(std::integral_constant<int, 3>{});
}

template <typename T, int K, bool X3 = false>
bool launch_tconv(const ConvArgsT<T>& a0, const TileSetDev& pts, hipStream_t st) {
  constexpr int CC = X3 ? 64 : stage_channels(K, 1) * (4 / (int)sizeof(T));
  if (a0.filt_mc == nullptr || a0.c1 % CC != 0 || a0.c2 % CC != 0 || a0.cout % 32 != 0) return false;
  ConvArgsT<T> a = a0;
  a.xcd_fs = 0;
  const unsigned cap_p = (unsigned)(pts.n * pts.tiles_y * pts.tiles_x);
  const unsigned cap_out = (unsigned)(a.ts.n * a.ts.tiles_y * a.ts.tiles_x);
  const int cout = a.cout;
  const long long groups = (long long)cap_p * (cout / 32);
  const int nch = (a.c1 + a.c2) / CC;
  if (a.ws != nullptr && !a.refresh && groups <= 128 && nch >= 4) {
    a.ws_plane = (long long)a.ts.n * a.ts.h * a.ts.w * cout;
    int parts = 1;
    while (2 * parts <= 8 && 2 * parts <= nch && groups * (2 * parts) <= 256 && (long long)(2 * parts) * a.ws_plane <= a.ws_floats)
      parts *= 2;
    if (parts >= 2) {
      hipLaunchKernelGGL((k_tconv_mfma<T, K, 1, true, X3>), dim3(cap_p, cout / 32, parts), dim3(256), 0, st, a, pts);
      unsigned ny = (unsigned)((1024 + cap_out - 1) / cap_out);
      if (ny > (unsigned)(cout / 4)) ny = (unsigned)(cout / 4);
      if (ny < 1) ny = 1;
      hipLaunchKernelGGL(k_conv_split_finish<T>, dim3(cap_out, ny), dim3(256), 0, st, a, parts);
      return true;
    }
  }
  a.ws = nullptr;
  // (the 128-column kernel holds 4 phases x 2 blocks of accumulators and a four-column operand ring: in the three-term
  // form it would spill, so that form stops at 64 columns)
  if (!X3 && cout % 128 == 0 && (long long)cap_p * (cout / 128) >= 400)
    hipLaunchKernelGGL((k_tconv_mfma<T, K, 4, false, false>), dim3(cap_p, cout / 128), dim3(256), 0, st, a, pts);
  else if (cout % 64 == 0 && (long long)cap_p * (cout / 64) >= 400)
    hipLaunchKernelGGL((k_tconv_mfma<T, K, 2, false, X3>), dim3(cap_p, cout / 64), dim3(256), 0, st, a, pts);
  else
    hipLaunchKernelGGL((k_tconv_mfma<T, K, 1, false, X3>), dim3(cap_p, cout / 32), dim3(256), 0, st, a, pts);
  return true;
}

template <typename T>
int tconv2x_impl(const char* who, const void* x, const uint8_t* xmask, int c1, const void* x2,
                 const uint8_t* x2mask, int c2, int h_in, int w_in, const float* filter, const void* filter_mc,
                 int cin_total, int k, int cout, const mie_tileset* out, const mie_tileset* blocks,
                 void* out_delta, const void* addend, float* reservoir, int act_kind, float slope, bool refresh,
                 const float* bias, void* workspace, long long workspace_bytes, void* stream, bool x3 = false) {
  int rc = mie_check_tileset(out, who);
  if (rc != MIE_OK) return rc;
  rc = mie_check_tileset(blocks, who);
  if (rc != MIE_OK) return rc;
  MIE_REQUIRE(x != nullptr && filter != nullptr && filter_mc != nullptr && out_delta != nullptr, MIE_ERR_INVALID_ARG,
              "%s: NULL pointer (x, filter, filter_mc and the output are required)", who);
  MIE_REQUIRE(c1 > 0 && c2 >= 0 && cout > 0 && h_in > 0 && w_in > 0 && (long long)c1 + c2 <= cin_total,
              MIE_ERR_INVALID_ARG, "%s: sizes out of range (c1=%d c2=%d cin_total=%d cout=%d h=%d w=%d)", who, c1, c2,
              cin_total, cout, h_in, w_in);
  MIE_REQUIRE((x2 != nullptr) == (c2 > 0) && (x2 != nullptr || x2mask == nullptr), MIE_ERR_INVALID_ARG,
              "%s: x2, c2 and x2mask must be given together", who);
  MIE_REQUIRE(k == 3 || k == 5, MIE_ERR_UNSUPPORTED, "%s: kernel size %d not implemented (3, 5)", who, k);
  MIE_REQUIRE(!x3 || sizeof(T) == 4, MIE_ERR_INVALID_ARG, "%s: MIE_DTYPE_F32_BF16X3 is a form of fp32 deltas", who);
  const int chunk = x3 ? 64 : 128 / (int)sizeof(T);
  MIE_REQUIRE(c1 % chunk == 0 && c2 % chunk == 0 && cout % 32 == 0 && cin_total % (x3 ? 16 : 32 / (int)sizeof(T)) == 0,
              MIE_ERR_UNSUPPORTED, "%s: needs c1, c2 %% %d == 0 and cout %% 32 == 0 (c1=%d c2=%d cout=%d)", who, chunk,
              c1, c2, cout);
  MIE_REQUIRE(out->h == 2 * h_in && out->w == 2 * w_in && blocks->h == h_in && blocks->w == w_in && blocks->n == out->n,
              MIE_ERR_INVALID_ARG, "%s: the output tile set must be (%d,%d) and the block tile set (%d,%d); got (%d,%d), (%d,%d)",
              who, 2 * h_in, 2 * w_in, h_in, w_in, out->h, out->w, blocks->h, blocks->w);
  MIE_REQUIRE((long long)out->n * out->h * out->w < 0x7fffffffLL && (long long)out->n * h_in * w_in * (c1 > c2 ? c1 : c2) < (1LL << 40),
              MIE_ERR_CAPACITY, "%s: tensor too large", who);
  MIE_REQUIRE(mie_aligned(x, 16) && mie_aligned(x2, 16) && mie_aligned(filter_mc, 16) && mie_aligned(out_delta, 16) &&
                  mie_aligned(addend, 16) && mie_aligned(reservoir, 16) && mie_aligned(bias, 4) && mie_aligned(workspace, 16),
              MIE_ERR_INVALID_ARG, "%s: buffers must be 16-byte aligned (bias: 4)", who);
  MIE_REQUIRE(act_kind >= MIE_ACT_NONE && act_kind <= MIE_ACT_TANH, MIE_ERR_UNSUPPORTED, "%s: unknown activation %d", who,
              act_kind);
  MIE_REQUIRE(refresh || reservoir != nullptr || act_kind == MIE_ACT_NONE, MIE_ERR_INVALID_ARG,
              "%s: activation %d needs a reservoir", who, act_kind);
  MIE_REQUIRE(addend == nullptr || addend != out_delta, MIE_ERR_INVALID_ARG, "%s: addend must not alias out_delta", who);
  MIE_REQUIRE(x != out_delta && (x2 == nullptr || x2 != out_delta), MIE_ERR_INVALID_ARG,
              "%s: x / x2 must not alias the output", who);
  MIE_REQUIRE(workspace_bytes >= 0 && (workspace != nullptr || workspace_bytes == 0), MIE_ERR_INVALID_ARG,
              "%s: workspace size without a workspace", who);
  MIE_REQUIRE(workspace == nullptr || (workspace != out_delta && workspace != (void*)reservoir && workspace != x && workspace != x2),
              MIE_ERR_INVALID_ARG, "%s: workspace must not alias an operand", who);
  ConvArgsT<T> a;
  a.x = (const T*)x; a.xm = xmask; a.c1 = c1; a.x2 = (const T*)x2; a.x2m = x2mask; a.c2 = c2;
  a.h_in = h_in; a.w_in = w_in; a.filt = filter; a.cin_total = cin_total; a.filt_mc = (const T*)filter_mc;
  a.pad = k / 2; a.cout = cout; a.out = (T*)out_delta; a.res = reservoir; a.act = act_kind; a.slope = slope;
  a.addend = (const T*)addend; a.refresh = refresh ? 1 : 0; a.bias = bias;
  a.hid = 0; a.g_cpd = nullptr; a.g_cpm = nullptr; a.g_cpres = nullptr; a.g_cres = nullptr; a.g_dh = nullptr; a.g_dc = nullptr;
  a.ws = (float*)workspace; a.ws_floats = workspace_bytes / 4; a.ws_plane = 0; a.xcd_fs = 0; a.x3 = x3 ? 1 : 0;
  a.ts = mie_dev_tileset(out);
  const TileSetDev pts = mie_dev_tileset(blocks);
  bool ok;
  if constexpr (sizeof(T) == 4) {
    if (x3) ok = (k == 3) ? launch_tconv<T, 3, true>(a, pts, (hipStream_t)stream) : launch_tconv<T, 5, true>(a, pts, (hipStream_t)stream);
    else ok = (k == 3) ? launch_tconv<T, 3>(a, pts, (hipStream_t)stream) : launch_tconv<T, 5>(a, pts, (hipStream_t)stream);
  } else {
    ok = (k == 3) ? launch_tconv<T, 3>(a, pts, (hipStream_t)stream) : launch_tconv<T, 5>(a, pts, (hipStream_t)stream);
  }
  MIE_REQUIRE(ok, MIE_ERR_UNSUPPORTED, "%s: no kernel variant for c1=%d c2=%d cout=%d", who, c1, c2, cout);
  return mie_check_launch(who);
}

}  // namespace

extern "C" int mie_tconv2x_masked(const void* x, const uint8_t* xmask, int c1, const void* x2, const uint8_t* x2mask,
                                  int c2, int h_in, int w_in, const float* filter, const void* filter_mc,
                                  int cin_total, int k, int cout, const mie_tileset* out, const mie_tileset* blocks,
                                  void* out_delta, const void* addend, float* reservoir, int act_kind, float slope,
                                  int dtype, void* workspace, long long workspace_bytes, void* stream) {
  const char* who = "mie_tconv2x_masked";
  mie_clear_error();
  const bool x3 = dtype == MIE_DTYPE_F32_BF16X3;
  if (x3) dtype = MIE_DTYPE_F32;
  MIE_REQUIRE(dtype == MIE_DTYPE_F32 || dtype == MIE_DTYPE_BF16, MIE_ERR_UNSUPPORTED, "%s: unknown delta dtype %d", who, dtype);
  if (dtype == MIE_DTYPE_BF16)
    return tconv2x_impl<mie_bf16>(who, x, xmask, c1, x2, x2mask, c2, h_in, w_in, filter, filter_mc, cin_total, k, cout, out,
                                  blocks, out_delta, addend, reservoir, act_kind, slope, false, nullptr, workspace,
                                  workspace_bytes, stream);
  return tconv2x_impl<float>(who, x, xmask, c1, x2, x2mask, c2, h_in, w_in, filter, filter_mc, cin_total, k, cout, out, blocks,
                             out_delta, addend, reservoir, act_kind, slope, false, nullptr, workspace, workspace_bytes,
                             stream, x3);
}

extern "C" int mie_tconv2x_refresh(const void* x, int c1, const void* x2, int c2, int h_in, int w_in, const float* filter,
                                   const void* filter_mc, int cin_total, int k, int cout, const float* bias,
                                   const mie_tileset* out, const mie_tileset* blocks, void* out_dense, const void* addend,
                                   float* reservoir, int act_kind, float slope, int dtype, void* stream) {
  const char* who = "mie_tconv2x_refresh";
  mie_clear_error();
  const bool x3 = dtype == MIE_DTYPE_F32_BF16X3;
  if (x3) dtype = MIE_DTYPE_F32;
  MIE_REQUIRE(dtype == MIE_DTYPE_F32 || dtype == MIE_DTYPE_BF16, MIE_ERR_UNSUPPORTED, "%s: unknown delta dtype %d", who, dtype);
  if (dtype == MIE_DTYPE_BF16)
    return tconv2x_impl<mie_bf16>(who, x, nullptr, c1, x2, nullptr, c2, h_in, w_in, filter, filter_mc, cin_total, k, cout, out,
                                  blocks, out_dense, addend, reservoir, act_kind, slope, true, bias, nullptr, 0, stream);
  return tconv2x_impl<float>(who, x, nullptr, c1, x2, nullptr, c2, h_in, w_in, filter, filter_mc, cin_total, k, cout, out, blocks,
                             out_dense, addend, reservoir, act_kind, slope, true, bias, nullptr, 0, stream, x3);
}
