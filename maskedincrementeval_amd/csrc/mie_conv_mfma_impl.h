// Kernel and launch templates of the matrix-core conv path, included by one translation unit per
// element type (mie_conv_mfma_f32.hip, mie_conv_mfma_bf16.hip) so that they compile in parallel.
//
// Masked conv on the matrix cores, gfx950: fp32 deltas with v_mfma_f32_32x32x2_f32, bf16 deltas
// with v_mfma_f32_32x32x16_bf16 (fp32 accumulation, fp32 reservoirs).  The two element types share
// one kernel: every operand access is a 16-byte access, which holds 4 fp32 or 8 bf16 channels, so
// the bf16 kernel is the fp32 kernel with twice the channels per LDS stage, per unit and per load.
// The text below gives the fp32 numbers.  A third form, X3, multiplies fp32 deltas on the bf16 instruction at fp32
// accuracy (three bf16 terms per value, six term products per multiply): it is described at the kernel template and
// is what fp32 deltas take by default wherever it exists.
//
// Work decomposition.  One 256-thread workgroup (4 waves) computes one active
// 8x8 output tile (M = 64 pixels) x CO_BLK output channels as an implicit GEMM
// over k = (input channel, tap):
//   * A (pixels x k): the input tile plus halo is staged in LDS, CC input
//     channels at a time, by all 256 threads with 16-byte loads of the NHWC
//     rows; pixels whose mask byte is 0 (or that lie outside the image) are
//     zero-filled without touching HBM.  The global loads of chunk c+1 are in
//     flight (in registers) while chunk c is multiplied; fp32 stride-1 tiles
//     also double-buffer the LDS copy, the others store it between two barriers.
//   * B (k x channels): units of the matrix-core filter copy (mie_pack_filter) are
//     read straight from L2 into a register ring, 16 bytes per lane (each value is
//     used by exactly one wave of the workgroup), 3 to 8 units ahead of the MFMAs
//     that consume them.
//   * The 4 waves split the workgroup's work WN ways over output channels and
//     WK = 4/WN ways over k (units = tap x 8-channel sub-chunk, round robin).
//     Layers with few tiles (33x44 bottleneck: 30 tiles) take WN=1, WK=4 so
//     that tiles x Cout/32 workgroups of 4 busy waves fill the chip; wide
//     layers take WN=4.  K-split partial sums meet in LDS and are added in a
//     fixed order (bit-reproducible).
//   * Epilogue: plain delta, or reservoir update + activation increment (values
//     fetched at kernel start in the k-split variants), or -- GATES -- the whole
//     ConvLSTM gate chain on the four gate columns of each hidden channel.
// A lane's operand layout: lanes 0-31 = the 32 pixels of an M block, the lane
// half selects 4 of the 8 channels of a sub-chunk, read as ONE ds_read_b128
// that feeds 4 k-steps (k-step j pairs channel j of the low half with channel
// 4+j of the high half; the B operand is loaded with the same pairing).  The
// LDS layout (pixel stride CC+4 dwords, row pitch 32 mod 64 dwords, half swap
// for stride 2) keeps the 16-byte reads of 16 neighbouring lanes on disjoint banks.
//
// What bounds it (measured on MI355X).  A register-only loop of the same MFMAs sustains 27.2 ns per
// v_mfma_f32_32x32x2_f32 and wave (64 cycles at 2.36 GHz; 152-155 TFLOP/s over the chip, constant or random
// operands alike) -- and 13.8 ns per v_mfma_f32_32x32x16_bf16 with constant operands but 20.6 ns (1.63 PFLOP/s,
// 0.65 of the nominal peak) with random ones: the bf16 rate is power-limited by the data.  In this kernel a
// 3x3 chunk of 72 MFMAs per wave takes 2.92 us = 40.6 ns per MFMA (one workgroup per CU, 3x3 256->256 at
// 33x44), a 5x5 chunk of 200 about 6.2 us = 31 ns.  Builds with parts of the loop compiled out (timing only)
// put the 3x3 kernel at 28.8 us complete, 27.6 without the A reads from LDS, 24.3 without any load, store or
// barrier in the loop; of those 24.3 us, 5.6 are tile pick, first staging round trip and epilogue.  The
// chunk hand-over, the B prefetch depth, the staging depth (64 channels per chunk), 8-wave workgroups, a
// third resident workgroup per CU (registers cut to fit) and splitting the contraction of the decoder convs
// over two or four workgroups were each built and measured: none moved a layer by more than 2 %, the last
// three for the worse.  Launches of a few workgroups per CU stay quantised: ceil(workgroups / 256) rounds.
// The X3 form does the same 3x3 chunk's work in 54 MFMAs of 32 cycles, 0.95 us, and takes 2.4 us for it: with one wave
// per SIMD nothing overlaps that wave's own staging work (88 VALU instructions to split a chunk's values, address
// arithmetic, waits -- the load counter is in order, so a filter prefetch behind the staging loads waits for them).
// A three-chunk software pipeline with two staging register sets changed nothing (19.8 us either way) and was removed;
// so were two extra waves that did all the staging with loads in flight four chunks ahead (chunk 2.2 -> 1.9 us, but a
// longer head: 20.8 -> 20.5 us).  With every filter load and LDS read of the loop made cache-resident on top of that
// (timing only) the chunk still takes 1.5 us: the staging latency is 0.3 us of it, all memory effects 0.7 us.
#pragma once
#include "mie_conv.h"
#include <stdlib.h>
#include <type_traits>

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
#ifndef MIE_PIPE
#define MIE_PIPE 1
#endif

// Build-time instrumentation (-DMIE_WG_PROFILE, measurement builds only): thread 0 of every workgroup
// records the 100 MHz device clock at the stages of its life into a buffer handed over with
// mie_set_profile_buffer, 16 slots per workgroup (slot 15 = number of stamps).  Compiled out otherwise.
#ifdef MIE_WG_PROFILE
static __device__ long long* mie_prof_buf;       // set by mie_set_profile_buffer (measurement builds only)
#define MIE_STAMP(k)                                                                                   \
  do {                                                                                                 \
    if (mie_prof_buf != nullptr && threadIdx.x == 0 && (k) < 15) {                                     \
      long long* slot_ = mie_prof_buf + (((long long)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * 16; \
      slot_[(k)] = (long long)wall_clock64();                                                          \
      if ((k) == 0) slot_[12] = (long long)clock64();                                                  \
      if ((k) == 14) slot_[13] = (long long)clock64();                                                 \
      slot_[15] = (k) + 1;                                                                             \
    }                                                                                                  \
  } while (0)
#else
#define MIE_STAMP(k) do { } while (0)
#endif

// fp32 channels staged in LDS per chunk (bf16: twice as many), by kernel size and stride, bounded
// by 64 KB of LDS.  Stride 1 double-buffers the staged tile of (7+K)^2 pixels.  Stride 2 tiles
// are (14+K)^2 pixels: they are single-buffered (the next chunk waits in registers and is
// stored between two barriers), which affords the same depth as stride 1 -- and with it the
// 4-way k-split that fills the chip on planes of a few dozen tiles; HALF is the shallower
// variant for channel counts that are not a multiple of the full depth.
__host__ __device__ constexpr int stage_channels(int K, int S, bool HALF = false) {
  return ((K <= 5) ? 32 : 16) / (HALF ? 2 : 1);
}
// bf16 tiles are single-buffered at stride 1 as well: a bf16 workgroup spends a few microseconds on
// the matrix cores, so what hides its latencies is the number of workgroups resident on the CU (LDS
// per workgroup halves), not the overlap inside one (measured: +10 % on the 8x480x640 decoder conv).
__host__ __device__ constexpr int stage_buffers(int S, int elem_size) { return (S == 1 && elem_size == 4) ? 2 : 1; }

// LDS dwords per row of the staged input tile.  The 16-byte operand reads of 16 neighbouring lanes
// (8 pixels of one tile row and of the next) must fall on 64 distinct banks: the pixel stride
// (CC + 4 dwords) spreads one row over every other group of 4 banks, and a row pitch of
// 32 (mod 64) dwords puts the next row on the groups in between (stride 1).  For stride 2 the
// pixel stride doubles and every row falls on the same bank groups whatever the pitch; there
// the two 16-byte halves of a unit are swapped in every other pair of input rows instead
// (`swz` below), which moves the neighbouring tile row by 4 banks.
__host__ __device__ constexpr int row_pitch_dw(int it, int ls_dw, int s) {
  int rp = it * ls_dw;
  if (s == 1)
    while (rp % 64 != 32) rp += 4;
  return rp;
}

// Ring size of the B-operand prefetch: the smallest divisor of the units per chunk that is
// at least 4, so that ring slot (unit % ring) means the same registers in every chunk.
__host__ __device__ constexpr int ring_size(int upc, int least = 4) {
  for (int r = least; r < upc; ++r)
    if (upc % r == 0) return r;
  return upc;
}

// Unit positions per chunk for the k-split over taps: at least n, padded until the ring size is at most 6
// (the extra positions hold no unit for any wave and compile to nothing).
__host__ __device__ constexpr int pad_units(int n) {
  while (ring_size(n) > 6) ++n;
  return n;
}

typedef float v4f __attribute__((ext_vector_type(4)));

// Waves per SIMD the register allocation must leave room for.  The stride-2 5x5 bf16 kernels stage a 19x19 tile
// (52 KB of LDS: three workgroups fit a CU) and spend two thirds of a workgroup's life outside the MFMA loop
// (tile pick, mask bytes, the one staging round trip, a 128-column epilogue), so a third resident workgroup
// is what fills the matrix cores; their natural allocation (172 registers) stops at two.
#ifndef MIE_S2_WAVES
#define MIE_S2_WAVES 3
#endif
__host__ __device__ constexpr int conv_min_waves(int elem_size, int K, int S, bool HALF, bool GATES, bool UP, bool SPLIT,
                                                 bool X3) {
  if (X3) return 2;      // 64 accumulator registers: the three-term kernels sit at the edge of two waves per SIMD
  return (elem_size == 2 && S == 2 && K == 5 && !HALF && !GATES && !UP && !SPLIT) ? MIE_S2_WAVES : 1;
}

// One unit of the contraction on the matrix core: the 16 bytes of A and of B a lane holds.
__device__ __forceinline__ void mma_unit(v16f& acc, const float4& av, const float4& bv, float) {
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.x, bv.x, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.y, bv.y, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.z, bv.z, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.w, bv.w, acc, 0, 0, 0);
}
__device__ __forceinline__ void mma_unit(v16f& acc, const float4& av, const float4& bv, mie_bf16) {
  const v4f a4 = {av.x, av.y, av.z, av.w}, b4 = {bv.x, bv.y, bv.z, bv.w};
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(mie_bf16x8, a4),
                                                __builtin_bit_cast(mie_bf16x8, b4), acc, 0, 0, 0);
}

// The same for the two pixel blocks of a tile against one B operand, the k-steps of the two accumulators
// interleaved: consecutive MFMAs are independent, so none waits for the result of the one before it.
__device__ __forceinline__ void mma_unit2(v16f& acc0, v16f& acc1, const float4& a0, const float4& a1, const float4& bv, float) {
  acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.x, bv.x, acc0, 0, 0, 0);
  acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.x, bv.x, acc1, 0, 0, 0);
  acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.y, bv.y, acc0, 0, 0, 0);
  acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.y, bv.y, acc1, 0, 0, 0);
  acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.z, bv.z, acc0, 0, 0, 0);
  acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.z, bv.z, acc1, 0, 0, 0);
  acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.w, bv.w, acc0, 0, 0, 0);
  acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.w, bv.w, acc1, 0, 0, 0);
}
__device__ __forceinline__ void mma_unit2(v16f& acc0, v16f& acc1, const float4& a0, const float4& a1, const float4& bv, mie_bf16) {
  mma_unit(acc0, a0, bv, mie_bf16());
  mma_unit(acc1, a1, bv, mie_bf16());
}

// X3 (fp32 deltas multiplied as three bf16 terms each): v = hi + mid + lo with every term rounded to nearest
// even, so |mid| <= 2^-9 |v|, |lo| <= 2^-18 |v| and the three terms carry all 24 bits of v.  The six products
// hi*hi, hi*mid, mid*hi, hi*lo, mid*mid, lo*hi are exact in the fp32 accumulator's input; what is left out
// (mid*lo, lo*mid, lo*lo) is at most 2^-23 of |a*b| and typically 2^-26 (an fp32 multiply-add rounds at 2^-24); the
// measured error of whole convs against fp64 is 0.6-0.8 of the fp32 instruction's in the same decomposition.  (Non-finite values do
// not survive the split: inf - inf is NaN.)
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 mie_bf16x2 __attribute__((ext_vector_type(2)));
// two values at a time: one packed conversion per term, the bf16 pair widened again with a shift and a mask
__device__ __forceinline__ void split3_pair(float f0, float f1, float& p0, float& p1, float& p2) {
  const v2f v = {f0, f1};
  const mie_bf16x2 hi = __builtin_convertvector(v, mie_bf16x2);
  const unsigned uh = __builtin_bit_cast(unsigned, hi);
  const v2f r1 = {f0 - __builtin_bit_cast(float, uh << 16), f1 - __builtin_bit_cast(float, uh & 0xffff0000u)};
  const mie_bf16x2 mid = __builtin_convertvector(r1, mie_bf16x2);
  const unsigned um = __builtin_bit_cast(unsigned, mid);
  const v2f r2 = {r1[0] - __builtin_bit_cast(float, um << 16), r1[1] - __builtin_bit_cast(float, um & 0xffff0000u)};
  const mie_bf16x2 lo = __builtin_convertvector(r2, mie_bf16x2);
  p0 = __builtin_bit_cast(float, hi);
  p1 = __builtin_bit_cast(float, mid);
  p2 = __builtin_bit_cast(float, lo);
}
__device__ __forceinline__ void split3(const float (&f)[8], float4 (&pl)[3]) {
  split3_pair(f[0], f[1], pl[0].x, pl[1].x, pl[2].x);
  split3_pair(f[2], f[3], pl[0].y, pl[1].y, pl[2].y);
  split3_pair(f[4], f[5], pl[0].z, pl[1].z, pl[2].z);
  split3_pair(f[6], f[7], pl[0].w, pl[1].w, pl[2].w);
}
// One unit (16 input channels of a tap) of the X3 contraction for the two pixel blocks of a tile: six bf16 MFMAs
// per block.  The three large products (hi*hi, mid*hi, hi*mid) and the three small ones (lo*hi, mid*mid, hi*lo, 2^-16 of
// the first) go to accumulators of their own, added in the epilogue: four independent chains, so that no MFMA
// waits for the one issued just before it, and the small terms are summed among themselves.
__device__ __forceinline__ void mma_unit2_x3(v16f& acc0, v16f& acc1, v16f& sm0, v16f& sm1, const float4 (&a0)[3],
                                             const float4 (&a1)[3], const float4 (&b)[3]) {
  mma_unit(acc0, a0[0], b[0], mie_bf16()); mma_unit(acc1, a1[0], b[0], mie_bf16());
  mma_unit(sm0, a0[2], b[0], mie_bf16());  mma_unit(sm1, a1[2], b[0], mie_bf16());
  mma_unit(acc0, a0[1], b[0], mie_bf16()); mma_unit(acc1, a1[1], b[0], mie_bf16());
  mma_unit(sm0, a0[1], b[1], mie_bf16());  mma_unit(sm1, a1[1], b[1], mie_bf16());
  mma_unit(acc0, a0[0], b[1], mie_bf16()); mma_unit(acc1, a1[0], b[1], mie_bf16());
  mma_unit(sm0, a0[0], b[2], mie_bf16());  mma_unit(sm1, a1[0], b[2], mie_bf16());
}

// One 16-byte slot of delta elements <-> fp32 values (4 of them, or 8 for bf16).
__device__ __forceinline__ void slot_to_f32(const float4& raw, float (&f)[4], float) {
  f[0] = raw.x; f[1] = raw.y; f[2] = raw.z; f[3] = raw.w;
}
__device__ __forceinline__ void slot_to_f32(const float4& raw, float (&f)[8], mie_bf16) {
  const v4f r4 = {raw.x, raw.y, raw.z, raw.w};
  const mie_bf16x8 b = __builtin_bit_cast(mie_bf16x8, r4);
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = (float)b[e];
}
__device__ __forceinline__ float4 f32_to_slot(const float (&f)[4], float) { return make_float4(f[0], f[1], f[2], f[3]); }
__device__ __forceinline__ float4 f32_to_slot(const float (&f)[8], mie_bf16) {
  mie_bf16x8 b;
#pragma unroll
  for (int e = 0; e < 8; ++e) b[e] = (mie_bf16)f[e];
  const v4f r4 = __builtin_bit_cast(v4f, b);
  return make_float4(r4[0], r4[1], r4[2], r4[3]);
}

// The gate chain of one item of a gates conv -- pixel `pix`, four adjacent hidden channels whose state values start at
// element `ho` and whose 16 gate columns start at element `go` of the gate reservoir -- given the conv sums dg of those
// columns: reservoirs updated, state deltas written.
template <typename T>
__device__ __forceinline__ void conv_gates_item(const ConvArgsT<T>& a, long long pix, long long ho, long long go, const float4 (&dg)[4]) {
  const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
  float4 rr[4];
  float4* gr = reinterpret_cast<float4*>(a.res + go);
#pragma unroll
  for (int j = 0; j < 4; ++j) rr[j] = gr[j];
  const bool has_cp = a.g_cpd != nullptr && (a.g_cpm == nullptr || a.g_cpm[pix]);
  const float4 dP4 = has_cp ? mie_ld4(a.g_cpd, ho) : zero4;
  const float4 cp4 = *reinterpret_cast<const float4*>(a.g_cpres + ho);
  const float4 cc4 = *reinterpret_cast<const float4*>(a.g_cres + ho);
  float cp[4] = {cp4.x, cp4.y, cp4.z, cp4.w}, cc[4] = {cc4.x, cc4.y, cc4.z, cc4.w};
  const float dP[4] = {dP4.x, dP4.y, dP4.z, dP4.w};
  float dh[4], dc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    mie_lstm_gate_chain(rr[j].x, rr[j].y, rr[j].z, rr[j].w, dg[j].x, dg[j].y, dg[j].z, dg[j].w, cp[j], dP[j], cc[j],
                        dh[j], dc[j]);
    gr[j] = rr[j];
  }
  if (has_cp) *reinterpret_cast<float4*>(a.g_cpres + ho) = make_float4(cp[0], cp[1], cp[2], cp[3]);
  *reinterpret_cast<float4*>(a.g_cres + ho) = make_float4(cc[0], cc[1], cc[2], cc[3]);
  mie_st4(a.g_dh, ho, make_float4(dh[0], dh[1], dh[2], dh[3]));
  mie_st4(a.g_dc, ho, make_float4(dc[0], dc[1], dc[2], dc[3]));
}

// UP: the conv input is up2x(x + x2), the bilinear x2 up-sampling of the sum of two deltas given at
// half resolution (x2 optional), and is never formed in memory: per chunk the 8x8 block of source
// pixels a tile's 12x12 input window blends is summed into LDS (fp32), and the staged tile is expanded
// from there.  5x5, stride 1, pad 2 only; a.h_in / a.w_in are the up-sampled size.
//
// SPLIT: launches with very few tiles (a 16x16 plane is 4 of them) leave most CUs idle.  The staged
// chunks of every (tile, slab) are then split over gridDim.z workgroups; each writes its partial sums,
// fp32 and unactivated, into its own plane of the workspace (a.ws, laid out like the output), and
// k_conv_split_finish adds the planes in a fixed order and runs the epilogue.  Only the 32-channel
// slab kernels (WN = 1) have this form.
//
// X3 (fp32 deltas only): the contraction runs on the bf16 matrix-core instruction at fp32 accuracy.  Every staged
// input value and every filter value is split into three bf16 terms (split3; the filter once, by
// mie_pack_filter); the staged tile is three bf16 planes in LDS, a unit is 16 input channels of a tap, and
// its six significant term products are six v_mfma_f32_32x32x16_bf16 per pixel block -- 6 x 32 cycles for what
// eight v_mfma_f32_32x32x2_f32 take 8 x 64 cycles to do.  Chunks of 32 channels (two units per tap; stride 2, whose
// staged tile is four times the size: 16 channels, one unit per tap); where the k-split has more waves than a tap
// has units it is over (sub-chunk, tap class).  Global loads, masks, epilogue: fp32.
template <typename T, int K, int S, int WN, int NB, bool HALF, bool GATES = false, bool UP = false, bool SPLIT = false,
          bool X3 = false>
// (Build with -mllvm -pragma-unroll-threshold=65536: the unit loop of the 128-column 5x5 / 7x7 kernels is 100 / 196
// positions long, and where the compiler refuses to unroll it the operand ring is indexed at run time and lands in
// scratch memory -- a factor of three in time.)
__global__ __launch_bounds__(256, conv_min_waves((int)sizeof(T), K, S, HALF, GATES, UP, SPLIT, X3)) void k_conv_mfma(ConvArgsT<T> a) {
  static_assert(!X3 || (sizeof(T) == 4 && !HALF && (K == 3 || K == 5)), "X3: fp32 deltas, 3x3 / 5x5");
  using TL = std::conditional_t<X3, mie_bf16, T>;            // element type in LDS and on the matrix cores
  constexpr int PL = X3 ? 3 : 1;                             // operand planes (terms per value)
  constexpr int GPS = X3 ? 2 : 1;                            // 16-byte global loads per staging slot
  constexpr int NBUF = X3 ? ((K == 3 && S == 1) ? 2 : 1) : stage_buffers(S, (int)sizeof(T));
  constexpr int EPS = 16 / (int)sizeof(TL);                  // elements per 16-byte slot (4 / 8)
  constexpr int SUB = 2 * EPS;                               // channels per unit (8 / 16)
  constexpr int WK = 4 / WN;
  constexpr int IT = 7 * S + K;                              // input tile edge incl. halo
  constexpr int CC = X3 ? (S == 2 ? 16 : 32) : stage_channels(K, S, HALF) * (4 / (int)sizeof(T));   // channels per LDS stage
  constexpr int LS = CC + EPS;                               // LDS elements per staged pixel
  constexpr int NPIX = IT * IT;
  constexpr int Q4 = CC / EPS;                               // 16-byte slots per pixel
  constexpr int NSLOT = NPIX * Q4;
  constexpr int NLD = (NSLOT + 255) / 256;                   // staging slots per thread
  constexpr int RP = row_pitch_dw(IT, LS * (int)sizeof(TL) / 4, S) * 4 / (int)sizeof(TL);   // elements per tile row
  constexpr int STAGE = IT * RP;                             // elements per plane of a staging buffer
  constexpr int NQ = CC / SUB;                               // sub-chunks (units per tap) per stage
  // k-split: over whole sub-chunks (every wave takes NQW of them, for every tap), or -- more waves than sub-chunks,
  // X3 only -- one sub-chunk and every TP-th tap per wave (the last position of a chunk is then empty for some waves)
  constexpr bool TPAR = WK > NQ;
  static_assert(TPAR ? (X3 && WK % NQ == 0) : (NQ % WK == 0), "the k-split is over whole sub-chunks, or over taps");
  constexpr int TP = TPAR ? WK / NQ : 1;                     // tap classes
  constexpr int NQW = TPAR ? 1 : NQ / WK;                    // sub-chunks per wave
  constexpr int UPC = TPAR ? pad_units((K * K + TP - 1) / TP) : K * K * NQW;   // unit positions per chunk and wave
  constexpr int RING = (X3 && ring_size(UPC) > 6) ? ring_size(UPC, 3) : ring_size(UPC);   // B operand ring (divides UPC)
  constexpr int PD = RING - 1;                               // prefetch distance in units
  constexpr int CO_BLK = 32 * NB * WN;
  constexpr int RED = WK * 64 * CO_BLK;                      // every wave parks its accumulators here for the epilogue
  constexpr int STAGE_F = NBUF * PL * STAGE * (int)sizeof(TL) / 4;  // the staging buffers, in floats
  constexpr int LOS = CC;                                    // floats per source pixel in LDS
  constexpr int LO_F = UP ? 64 * LOS : 0;                    // fp32 sums of the 8x8 source block, CC channels
  static_assert(!UP || (S == 1 && K == 5 && !GATES), "the up-sampling variant is the 5x5 stride-1 conv");
  // the k-split reduction of the epilogue reuses the staging buffers and the source block
  constexpr int SMEM = (STAGE_F + LO_F > RED) ? STAGE_F + LO_F : RED;
  static_assert(SMEM * 4 <= 65536, "LDS budget");
  __shared__ __attribute__((aligned(16))) float smem[SMEM];
  TL* const sbuf = reinterpret_cast<TL*>(smem);
  float* const s_lo = smem + STAGE_F;

  // (tile-list position, slab, part) of this workgroup.  Each of the 8 XCDs has an L2 of its own and the
  // hardware hands workgroups to the XCDs round robin in launch order (x fastest); with a.xcd_fs > 0 the
  // grid's x extent is a multiple of 8, so the XCD of a workgroup is blockIdx.x % 8, and the launch order
  // is permuted.  The live (tile, slab) pairs are put in the order (slab group, tile, slab within the
  // group) -- a.xcd_fs groups of slabs, tiles in list order, i.e. along the rows of the image -- and each
  // XCD takes a contiguous eighth of it, in that order.  A slab of the filter then reaches 8 / xcd_fs
  // L2s instead of all 8, an input tile about xcd_fs of them, once, for all slabs of the group at a
  // time, and neighbouring tiles, which share their halo, meet in one L2 (measured on the 5x5 256->128
  // conv at 66x88: 65 -> 31 MB fetched per launch).  Active and stale tiles are dealt out separately
  // (a stale tile costs next to nothing); the shares depend on their numbers, read from the tile set
  // (one more dependent load at the start of a workgroup: measured, it costs nothing even on launches
  // of a few dozen workgroups), and idle positions of the capacity-sized grid fall off the end.
  // (For the SPLIT launches the same idea, one filter slice per XCD, was measured: no gain.)
  const int entry_zero = conv_args_entry_zero(a);      // every line of the argument block, fetched in one batch
  MIE_STAMP(0);
  int bx = blockIdx.x + entry_zero, by = blockIdx.y;
  const int bz = SPLIT ? (int)blockIdx.z : 0;
  int n, y0, x0, tk;
  if (!SPLIT && a.xcd_fs > 0) {
    const int cap = a.ts.n * a.ts.tiles_y * a.ts.tiles_x;
    const int n_act = a.ts.counts[MIE_CNT_ACTIVE], n_st = a.ts.counts[MIE_CNT_STALE];
    if (n_act < 0 || n_st < 0 || n_act > cap || n_st > cap) return;
    const int ns = (int)gridDim.y;
    const int w_act = n_act * ns, w_st = n_st * ns;          // live workgroups
    const int c_act = (w_act + 7) >> 3, c_st = (w_st + 7) >> 3;   // per XCD
    const int xcd = bx & 7;
    const int slot = by * ((int)gridDim.x >> 3) + (bx >> 3);      // launch order within the XCD
    const int spg = ns / a.xcd_fs;                           // slabs per group
    int v, tiles_of_kind;
    const bool active = slot < c_act;
    if (active) {
      v = xcd * c_act + slot;
      if (v >= w_act) return;
      tiles_of_kind = n_act;
    } else {
      if (slot - c_act >= c_st) return;
      v = xcd * c_st + (slot - c_act);
      if (v >= w_st) return;
      tiles_of_kind = n_st;
    }
    const int per_group = tiles_of_kind * spg;
    const int sg = v / per_group, r = v - sg * per_group;
    const int t = r / spg;
    by = sg * spg + (r - t * spg);
    bx = active ? t : n_act + t;
    tk = mie_pick_tile_loaded(a.ts, bx, active ? a.ts.tiles[t] : 0, n_act, n_st, n, y0, x0);
  } else {
    tk = mie_pick_tile(a.ts, bx, n, y0, x0);
  }
  if (tk == 0) return;
  MIE_STAMP(1);
  const int tid = threadIdx.x;
  // wave index as a scalar: everything derived from it (k-split, channel slab) stays in SGPRs
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int wn = wave % WN, wk = wave / WN;
  const int co0 = by * CO_BLK;
  const int hout = a.ts.h, wout = a.ts.w;
  const int cout = a.cout;

  static_assert(!SPLIT || (WN == 1 && !GATES), "the split form is a 32-channel slab kernel (the gates conv splits as a plain conv)");
  if (SPLIT && tk == 2) return;      // stale tiles are zeroed by k_conv_split_finish
  if (GATES && tk == 2) {  // stale tile: zero the hidden / cell deltas of this workgroup's hidden channels
    constexpr int HG = CO_BLK / 16;          // groups of four hidden channels
    for (int idx = tid; idx < 64 * HG; idx += 256) {
      const int p = idx / HG, g4 = idx - p * HG;
      const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
      if (oy < hout && ox < wout) {
        const long long o = (((long long)n * hout + oy) * wout + ox) * a.hid + co0 / 4 + 4 * g4;
        mie_st4(a.g_dh, o, make_float4(0.f, 0.f, 0.f, 0.f));
        mie_st4(a.g_dc, o, make_float4(0.f, 0.f, 0.f, 0.f));
      }
    }
    return;
  }
  if (tk == 2) {  // stale tile: zero this workgroup's channel slab
    for (int idx = tid; idx < 16 * CO_BLK; idx += 256) {       // groups of four channels
      const int p = idx / (CO_BLK / 4), col = 4 * (idx - p * (CO_BLK / 4));
      const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
      if (oy < hout && ox < wout)
        mie_st4(a.out, (((long long)n * hout + oy) * wout + ox) * cout + co0 + col, make_float4(0.f, 0.f, 0.f, 0.f));
    }
    return;
  }

  // Epilogue (all but the gate chain): every wave parks its accumulators in LDS, and a thread then owns groups of
  // four adjacent output channels of a pixel -- 16-byte reads of the k-split partial sums, 16-byte reservoir
  // accesses, 16- / 8-byte delta accesses.  A thread's share of the output is fixed by its index, so in the k-split
  // fp32 kernels the reservoir / addend values are fetched right away and have the whole contraction to arrive.
  constexpr int QPP = CO_BLK / 4;                            // groups of four channels per pixel
  constexpr int PER = GATES ? 1 : 64 * QPP / 256;            // groups per thread
  constexpr int PB = PER > 4 ? 4 : PER;                      // groups per pass of the epilogue (registers)
  long long e_off[PB];
  int e_co[PB];
  bool e_ok[PB], e_live[PB];
  float4 e_r0[PB], e_add[PB];
  // bit g: group g of this thread lies on a pixel of the output pixel mask.  Elsewhere in an active tile the sums are
  // exactly zero: no reservoir access, a zero delta.  (The bytes are asked for here, long before the epilogue needs them.)
  unsigned live_bits = 0u;
  if (!GATES && !SPLIT) {
#pragma unroll
    for (int g = 0; g < PER; ++g) {
      const int p = (tid + 256 * g) / QPP;
      const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
      if (oy < hout && ox < wout && (a.refresh || a.ts.pixmask[((long long)n * hout + oy) * wout + ox] != 0)) live_bits |= 1u << g;
    }
  }
  // (bf16: a workgroup's contraction is too short to be worth the registers that hold these values
  // through it -- they cost a resident workgroup per CU -- so they are fetched after it instead; the same
  // holds for the 128-column slabs, whose threads own 8 groups.)
  constexpr bool EARLY = sizeof(T) == 4 && WK > 1 && !(X3 && K == 5);
  static_assert(!EARLY || PER == PB, "the early fetch covers a thread's whole share");
  auto epilogue_fetch = [&](int h0) {
#pragma unroll
    for (int i = 0; i < PB; ++i) {
      const int idx = tid + 256 * (h0 + i);
      const int p = idx / QPP, col = 4 * (idx - p * QPP);
      const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
      e_ok[i] = oy < hout && ox < wout;
      e_live[i] = SPLIT ? e_ok[i] : ((live_bits >> (h0 + i)) & 1u) != 0;
      e_off[i] = (((long long)n * hout + oy) * wout + ox) * a.cout + co0 + col;
      e_co[i] = co0 + col;
    }
    if (!SPLIT) conv_epilogue_load4<T, PB>(a, e_off, e_live, e_r0, e_add);
  };
  if (!GATES && EARLY && !SPLIT) epilogue_fetch(0);

  v16f acc[2][NB];
  v16f accs[X3 ? 2 : 1][X3 ? NB : 1];      // X3: the small term products
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        acc[mb][nb][r] = 0.f;
        if (X3) accs[mb][nb][r] = 0.f;
      }

  // ---- per-thread staging plan: which pixels / float4 slots this thread copies -------------
  const int iy0 = y0 * S - a.pad, ix0 = x0 * S - a.pad;
  int st_po[NLD];       // linear input pixel index
  int st_lds[NLD];      // LDS element offset of the slot
  int st_c4[NLD];       // channel offset of the slot inside the chunk
  unsigned ok1 = 0u, ok2 = 0u;   // slot readable from x / x2 (inside the image, pixel mask set)
  unsigned inb = 0u;             // slot inside the image
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int slot = tid + 256 * i;
    const int pix = slot / Q4, q4 = slot - pix * Q4;
    const int lrow = pix / IT;
    const int swz = (S == 2) ? ((lrow >> 1) & 1) : 0;
    st_lds[i] = lrow * RP + (pix - lrow * IT) * LS + EPS * (q4 ^ swz);
    st_c4[i] = EPS * q4;
    st_po[i] = 0;
    if (!UP && slot < NSLOT) {
      const int iy = iy0 + pix / IT, ix = ix0 + pix % IT;
      if (iy >= 0 && iy < a.h_in && ix >= 0 && ix < a.w_in) {
        st_po[i] = (n * a.h_in + iy) * a.w_in + ix;
        inb |= 1u << i;
      }
    }
  }
  const int nch1 = (a.c1 + CC - 1) / CC;
  const int nch = nch1 + ((!UP && a.x2 != nullptr) ? (a.c2 + CC - 1) / CC : 0);

  // UP: the source block.  Rows iy0 .. iy0+11 of the up-sampled image (iy0 even) blend source rows
  // iy0/2 - 1 .. iy0/2 + 6; one 16-byte slot per (source pixel, channel group) and tensor.
  constexpr int NLO = UP ? (64 * Q4 + 255) / 256 : 1;
  const int h_lo = a.h_in >> 1, w_lo = a.w_in >> 1;
  const int lo_y0 = (iy0 >> 1) - 1, lo_x0 = (ix0 >> 1) - 1;
  int lo_po[NLO];
  unsigned lo_ok1 = 0u, lo_ok2 = 0u, lo_inb = 0u;
  float4 lo_a[NLO][GPS], lo_b[NLO][GPS];
  if (UP) {
#pragma unroll
    for (int i = 0; i < NLO; ++i) {
      const int slot = tid + 256 * i;
      const int lpix = slot / Q4;
      const int ly = lo_y0 + (lpix >> 3), lx = lo_x0 + (lpix & 7);
      lo_po[i] = 0;
      if (lpix < 64 && ly >= 0 && ly < h_lo && lx >= 0 && lx < w_lo) {
        lo_po[i] = (n * h_lo + ly) * w_lo + lx;
        lo_inb |= 1u << i;
      }
    }
  }

  // The pixel-mask bytes a workgroup needs are one more dependent round trip at its start (tile id -> mask
  // bytes -> input loads).  Where the contraction has at least four chunks, the loads of the FIRST chunk
  // therefore go out for every pixel inside the image, before the mask bytes are there (`first`), and the
  // masked pixels are zeroed when the bytes have arrived; from the second chunk on -- and in layers of fewer
  // chunks, where that would be a large share of the reads -- a masked pixel is not fetched at all.
  float4 st_reg[NLD][GPS];
  auto load_slots = [&](float4 (&regs)[NLD][GPS], int c, bool first) {
    const bool second = c >= nch1;
    const T* xin = second ? a.x2 : a.x;
    const int cs = second ? a.c2 : a.c1;
    const int ci0 = (second ? c - nch1 : c) * CC;
    const unsigned ok = first ? inb : (second ? ok2 : ok1);
    // The loads are unconditional in control flow (a branch around a load makes the compiler's
    // wait counters conservative: the first MFMAs of a chunk would then wait for the whole
    // global-memory latency of these loads).  Lanes whose pixel is masked or outside the image
    // all read one fixed, cache-resident address instead and get zeros selected afterwards,
    // so inactive pixels still cost no HBM traffic.
    const T* dummy = a.filt_mc;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const bool okb = (ok >> i) & 1u;
      const T* p = xin + (long long)st_po[i] * cs + ci0 + st_c4[i];
      p = okb ? p : dummy;
#pragma unroll
      for (int g = 0; g < GPS; ++g) {
        float4 v = *reinterpret_cast<const float4*>(p + 4 * g);
        v.x = okb ? v.x : 0.f; v.y = okb ? v.y : 0.f; v.z = okb ? v.z : 0.f; v.w = okb ? v.w : 0.f;
        regs[i][g] = v;
      }
    }
  };
  auto stage_load = [&](int c, bool first = false) {
    if constexpr (UP) {
      const T* dummy = a.filt_mc;
#pragma unroll
      for (int i = 0; i < NLO; ++i) {
        const int q4 = (tid + 256 * i) % Q4;
        const long long eo = (long long)lo_po[i] * a.c1 + c * CC + EPS * q4;
        const bool k1 = ((first ? lo_inb : lo_ok1) >> i) & 1u;
        const bool k2 = first ? (a.x2 != nullptr && ((lo_inb >> i) & 1u)) : ((lo_ok2 >> i) & 1u);
#pragma unroll
        for (int g = 0; g < GPS; ++g) {
          float4 v = *reinterpret_cast<const float4*>(k1 ? a.x + eo + 4 * g : dummy);
          float4 u = *reinterpret_cast<const float4*>(k2 ? a.x2 + eo + 4 * g : dummy);
          v.x = k1 ? v.x : 0.f; v.y = k1 ? v.y : 0.f; v.z = k1 ? v.z : 0.f; v.w = k1 ? v.w : 0.f;
          u.x = k2 ? u.x : 0.f; u.y = k2 ? u.y : 0.f; u.z = k2 ? u.z : 0.f; u.w = k2 ? u.w : 0.f;
          lo_a[i][g] = v;
          lo_b[i][g] = u;
        }
      }
      return;
    }
    load_slots(st_reg, c, first);
  };
  // one staged slot to LDS: as it is, or (X3) its eight fp32 values as three bf16 planes
  auto store_slot = [&](TL* dst, const float4 (&raw)[GPS]) {
    if constexpr (X3) {
      const float f[8] = {raw[0].x, raw[0].y, raw[0].z, raw[0].w, raw[1].x, raw[1].y, raw[1].z, raw[1].w};
      float4 pl[3];
      split3(f, pl);
#pragma unroll
      for (int q = 0; q < 3; ++q) *reinterpret_cast<float4*>(dst + q * STAGE) = pl[q];
    } else {
      *reinterpret_cast<float4*>(dst) = raw[0];
    }
  };
  auto store_slots = [&](const float4 (&regs)[NLD][GPS], int buf) {
    TL* dst = sbuf + buf * (PL * STAGE);
#pragma unroll
    for (int i = 0; i < NLD; ++i)
      if (tid + 256 * i < NSLOT) store_slot(dst + st_lds[i], regs[i]);
  };
  auto stage_store = [&](int buf) {
    TL* dst = sbuf + buf * (PL * STAGE);
    if constexpr (UP) {
      // x + x2 of the source block to LDS in fp32 (bit pattern zero = 0 in both element types) ...
#pragma unroll
      for (int i = 0; i < NLO; ++i) {
        const int slot = tid + 256 * i;
        const int lpix = slot / Q4, q4 = slot - lpix * Q4;
        float fa[EPS], fb[EPS];
        if constexpr (X3) {
          const float ta[8] = {lo_a[i][0].x, lo_a[i][0].y, lo_a[i][0].z, lo_a[i][0].w, lo_a[i][1].x, lo_a[i][1].y, lo_a[i][1].z, lo_a[i][1].w};
          const float tb[8] = {lo_b[i][0].x, lo_b[i][0].y, lo_b[i][0].z, lo_b[i][0].w, lo_b[i][1].x, lo_b[i][1].y, lo_b[i][1].z, lo_b[i][1].w};
#pragma unroll
          for (int e = 0; e < 8; ++e) fa[e] = ta[e], fb[e] = tb[e];
        } else {
          slot_to_f32(lo_a[i][0], fa, T());
          slot_to_f32(lo_b[i][0], fb, T());
        }
        if (lpix < 64) {
#pragma unroll
          for (int e = 0; e < EPS; e += 4)
            *reinterpret_cast<float4*>(&s_lo[lpix * LOS + q4 * EPS + e]) =
                make_float4(fa[e] + fb[e], fa[e + 1] + fb[e + 1], fa[e + 2] + fb[e + 2], fa[e + 3] + fb[e + 3]);
        }
      }
      __syncthreads();
      // ... and the staged tile blended from it; pixels outside the up-sampled image are the conv's zero padding.
      // The taps' LDS offsets and weights depend on the tile only, and the compiler computes them once
      // and keeps 40 registers alive through the contraction.  fp32 kernels have the registers to spare
      // (two workgroups per CU either way) and run 1.5 % faster for it; in the bf16 kernels they cost
      // one or two resident workgroups, so there an opaque zero makes them a per-chunk computation.  The three-term
      // kernels: the 32-column one would pass 256 registers and lose its second workgroup; the wider ones have the
      // room (252) and keep the values (decoder 0 of the 264x352 frame 73 -> 70 us).
      int opaque = 0;
      if (sizeof(T) == 2 || (X3 && WN == 1)) asm volatile("" : "+v"(opaque));
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const int slot = tid + 256 * i + opaque;
        if (slot >= NSLOT) continue;
        const int pix = slot / Q4, q4 = slot - pix * Q4;
        const int hy = iy0 + pix / IT, hx = ix0 + pix % IT;
        float o[EPS];
#pragma unroll
        for (int e = 0; e < EPS; ++e) o[e] = 0.f;
        if (hy >= 0 && hy < a.h_in && hx >= 0 && hx < a.w_in) {
          int r0, r1, q0, q1;
          float lr0, lr1, lq0, lq1;
          conv_up2x_coef(hy, h_lo, r0, r1, lr0, lr1);
          conv_up2x_coef(hx, w_lo, q0, q1, lq0, lq1);
          const float* v00 = s_lo + ((r0 - lo_y0) * 8 + (q0 - lo_x0)) * LOS + q4 * EPS;
          const float* v01 = s_lo + ((r0 - lo_y0) * 8 + (q1 - lo_x0)) * LOS + q4 * EPS;
          const float* v10 = s_lo + ((r1 - lo_y0) * 8 + (q0 - lo_x0)) * LOS + q4 * EPS;
          const float* v11 = s_lo + ((r1 - lo_y0) * 8 + (q1 - lo_x0)) * LOS + q4 * EPS;
#pragma unroll
          for (int e = 0; e < EPS; e += 4) {       // 16-byte LDS reads
            const float4 t00 = *reinterpret_cast<const float4*>(v00 + e), t01 = *reinterpret_cast<const float4*>(v01 + e);
            const float4 t10 = *reinterpret_cast<const float4*>(v10 + e), t11 = *reinterpret_cast<const float4*>(v11 + e);
            o[e] = conv_up2x_v(lr0, lr1, conv_up2x_h(lq0, lq1, t00.x, t01.x), conv_up2x_h(lq0, lq1, t10.x, t11.x));
            o[e + 1] = conv_up2x_v(lr0, lr1, conv_up2x_h(lq0, lq1, t00.y, t01.y), conv_up2x_h(lq0, lq1, t10.y, t11.y));
            o[e + 2] = conv_up2x_v(lr0, lr1, conv_up2x_h(lq0, lq1, t00.z, t01.z), conv_up2x_h(lq0, lq1, t10.z, t11.z));
            o[e + 3] = conv_up2x_v(lr0, lr1, conv_up2x_h(lq0, lq1, t00.w, t01.w), conv_up2x_h(lq0, lq1, t10.w, t11.w));
          }
        }
        const int lrow = pix / IT;
        TL* d = dst + lrow * RP + (pix - lrow * IT) * LS + EPS * q4;
        if constexpr (X3) {
          float4 pl[3];
          split3(o, pl);
#pragma unroll
          for (int q = 0; q < 3; ++q) *reinterpret_cast<float4*>(d + q * STAGE) = pl[q];
        } else {
          *reinterpret_cast<float4*>(d) = f32_to_slot(o, T());
        }
      }
      return;
    }
    store_slots(st_reg, buf);
  };

  // ---- operand addressing ------------------------------------------------------------------------
  // This wave multiplies sub-chunks q = q0w .. q0w+NQW-1 of every chunk.  A unit is one tap of
  // one sub-chunk: 8 input channels, of which this lane's half handles 4 (channel pairing see
  // the header).  Everything that depends on the unit index is a compile-time constant times
  // cout (B) or a compile-time LDS offset (A); the lane-dependent parts are loop invariant.
  const int q0w = TPAR ? wk % NQ : wk * NQW;
  const int par = TPAR ? wk / NQ : 0;                          // tap class of this wave (scalar)
  // (tap, sub-chunk) of unit position `unit`; with the k-split over taps the tap depends on the wave and the last
  // position may hold no unit (tap >= K*K): it then multiplies nothing and prefetches the last tap once more
  auto unit_tap = [&](int unit) { return TPAR ? unit * TP + par : unit / NQW; };
  auto unit_sub = [&](int unit) { return TPAR ? 0 : unit % NQW; };
  const int cob0 = co0 + wn * (32 * NB);                       // first column of this wave
  const int b_lane = (half * cout + l32) * EPS;                // lane part of the packed filter index
  int a_lane[2][2];                                            // lane part of the LDS index
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {
    const int p = mb * 32 + l32;
    const int rowcol = ((p >> 3) * S) * RP + ((p & 7) * S) * LS + SUB * q0w;
    // stride 2: tile row r reads input row 2r + ky, whose halves are swapped iff (r + ky/2) is odd
    const int h0 = (S == 2) ? (half ^ ((p >> 3) & 1)) : half;
    a_lane[mb][0] = rowcol + EPS * h0;
    a_lane[mb][1] = rowcol + EPS * (h0 ^ 1);
  }
  // filter row block of chunk c for this wave (c1 and c2 are multiples of CC: no partial chunks)
  auto chunk_b = [&](int c) -> const TL* {
    const bool second = c >= nch1;
    const int ci0 = (second ? c - nch1 : c) * CC;
    const int fb = second ? a.c1 : 0;
    return reinterpret_cast<const TL*>(a.filt_mc) +
           ((long long)((fb + ci0) / SUB + q0w) * (K * K) * (PL * 2) * cout + cob0) * EPS;
  };
  // Matrix-core filter copy: P[ci/8][tap][(ci%8)/4][co][ci%4] (fp32; 16 / 8 / 8 for bf16; X3: the bf16 layout with
  // the three term planes of a (block, tap) next to each other, P[ci/16][tap][term][(ci%16)/8][co][ci%8]).  The
  // k-steps of a unit are one 16-byte load per lane (and term), 512 contiguous bytes per half wave.
  float4 bring[RING][NB][PL];
  auto load_b = [&](const TL* ub, int unit, float4 (&bv)[NB][PL]) {
    if (TPAR && unit * TP >= K * K) return;          // padding position: no unit for any wave
    int tap = unit_tap(unit);                        // compile-time after unrolling, but for the k-split over taps
    const int qi = unit_sub(unit);
    if (TPAR && tap >= K * K) tap = K * K - 1;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int q = 0; q < PL; ++q)
        bv[nb][q] = *reinterpret_cast<const float4*>(
            ub + ((long long)(((qi * (K * K) + tap) * PL + q) * 2) * cout + nb * 32) * EPS + b_lane);
  };

  // All B loads below are unconditional: a conditional load would make the compiler's wait
  // counters conservative and collapse the prefetch distance.  After the last chunk the
  // "next chunk" pointer simply stays on the current one (a few redundant loads).
  // SPLIT: part blockIdx.z of gridDim.z takes a contiguous range of the chunks (the host keeps
  // gridDim.z <= nch, so no range is empty)
  const int c_lo = SPLIT ? bz * nch / (int)gridDim.z : 0;
  const int c_hi = SPLIT ? (bz + 1) * nch / (int)gridDim.z : nch;
  const TL* ub_cur = chunk_b(c_lo);
  const TL* ub_next = ub_cur;
  MIE_STAMP(2);
  const bool early = c_hi - c_lo >= 4;      // uniform over the workgroup
  if (early) stage_load(c_lo, true);
  // the pixel-mask bytes, behind the first chunk's loads (pixel 0 stands in for slots outside the image, so that
  // these loads are unconditional too)
  {
    const bool m1 = a.xm != nullptr, has2 = a.x2 != nullptr, m2 = has2 && a.x2m != nullptr;
    if constexpr (UP) {
#pragma unroll
      for (int i = 0; i < NLO; ++i) {
        const unsigned b = (lo_inb >> i) & 1u;
        const unsigned v1 = m1 ? (unsigned)(a.xm[lo_po[i]] != 0) : 1u;
        const unsigned v2 = m2 ? (unsigned)(a.x2m[lo_po[i]] != 0) : (has2 ? 1u : 0u);
        lo_ok1 |= (b & v1) << i;
        lo_ok2 |= (b & v2) << i;
      }
    } else {
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const unsigned b = (inb >> i) & 1u;
        const unsigned v1 = m1 ? (unsigned)(a.xm[st_po[i]] != 0) : 1u;
        const unsigned v2 = m2 ? (unsigned)(a.x2m[st_po[i]] != 0) : (has2 ? 1u : 0u);
        ok1 |= (b & v1) << i;
        ok2 |= (b & v2) << i;
      }
    }
  }
  if (!early) stage_load(c_lo);
#pragma unroll
  for (int i = 0; i < (PD > 0 ? PD : 1); ++i) load_b(ub_cur, i, bring[i % RING]);
  // zero what the first chunk's loads fetched of masked pixels
  if (!early) {
  } else if constexpr (UP) {
#pragma unroll
    for (int i = 0; i < NLO; ++i)
#pragma unroll
      for (int g = 0; g < GPS; ++g) {
        if (!((lo_ok1 >> i) & 1u)) lo_a[i][g] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (!((lo_ok2 >> i) & 1u)) lo_b[i][g] = make_float4(0.f, 0.f, 0.f, 0.f);
      }
  } else {
    const unsigned ok = (c_lo >= nch1) ? ok2 : ok1;
#pragma unroll
    for (int i = 0; i < NLD; ++i)
#pragma unroll
      for (int g = 0; g < GPS; ++g)
        if (!((ok >> i) & 1u)) st_reg[i][g] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
  stage_store(0);
  __syncthreads();
  MIE_STAMP(3);

  // A operand of unit `unit` from the staged chunk at `sin` (one 16-byte LDS read per pixel block).
  auto load_a = [&](const TL* sin, int unit, float4 (&dst)[2][PL]) {
    if (TPAR && unit * TP >= K * K) return;
    int tap = unit_tap(unit);
    const int qi = unit_sub(unit);
    if (TPAR && tap >= K * K) tap = K * K - 1;
    const int ky = tap / K, kx = tap - ky * K;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int q = 0; q < PL; ++q)
        dst[mb][q] = *reinterpret_cast<const float4*>(
            &sin[q * STAGE + a_lane[mb][(S == 2) ? ((ky >> 1) & 1) : 0] + ky * RP + kx * LS + SUB * qi]);
  };
  // the MFMAs of one unit position
  auto mma = [&](int unit, const float4 (&av)[2][PL], const float4 (&bv)[NB][PL]) {
    if (TPAR && (unit * TP >= K * K || unit_tap(unit) >= K * K)) return;     // uniform over the wave
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      if constexpr (X3) mma_unit2_x3(acc[0][nb], acc[1][nb], accs[0][nb], accs[1][nb], av[0], av[1], bv[nb]);
      else mma_unit2(acc[0][nb], acc[1][nb], av[0][0], av[1][0], bv[nb][0], T());
    }
  };

  // Double-buffered kernels fold the chunk hand-over into the contraction, so that the matrix cores run
  // through it:
  //   * the next chunk's addresses are computed and its global loads issued right after the MFMAs of the
  //     first unit (an opaque copy of the chunk index keeps the compiler from hoisting the ~70 address
  //     instructions in front of them, where they ran with the matrix cores idle);
  //   * its LDS stores go out under the unit before the last but one;
  //   * the barrier sits between the last two units: by then every wave holds the A operands of its last
  //     unit in registers, so the barrier, and the LDS read of the next chunk's first operands (a register
  //     set of their own) behind it, pass under the last unit's MFMAs.
  // Measured on MI355X this ordering is worth under 1 % against "loads at the top of the chunk, stores and
  // barrier at its end": what a chunk loses against its MFMA time is not the hand-over (see the header).
  constexpr bool PIPE = MIE_PIPE && NBUF == 2 && !UP && UPC >= 8;
  if constexpr (PIPE) {
    float4 av[2][2][PL], av0[2][PL];
    load_a(sbuf, 0, av0);
    for (int c = c_lo; c < c_hi; ++c) {
      const bool more = c + 1 < c_hi;
      const TL* sin = sbuf + ((c - c_lo) & 1) * (PL * STAGE);
      const TL* sin_next = sbuf + ((c - c_lo + 1) & 1) * (PL * STAGE);
#pragma unroll
      for (int i = 0; i < UPC; ++i) {
        if (PD > 0) {
          const int ip = i + PD;
          if (ip < UPC) load_b(ub_cur, ip, bring[ip % RING]);
          else load_b(ub_next, ip - UPC, bring[ip % RING]);
        }
        if (i + 1 < UPC) load_a(sin, i + 1, av[(i + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
        if (i == 0) mma(0, av0, bring[0]);
        else mma(i, av[i & 1], bring[i % RING]);
        __builtin_amdgcn_sched_barrier(0);
        if (i == 0) {
          int cn = __builtin_amdgcn_readfirstlane(more ? c + 1 : c);      // after the last chunk: redundant re-load, never stored
          asm volatile("" : "+s"(cn));
          ub_next = chunk_b(cn);
          stage_load(cn);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (i == UPC - 3) {
          if (more) stage_store((c - c_lo + 1) & 1);    // the other buffer: nobody reads it during this chunk
          __builtin_amdgcn_sched_barrier(0);
        }
        if (i == UPC - 2) {
          // every wave has its last operands of this chunk (the wait for them is part of the barrier)
          __syncthreads();
          load_a(sin_next, 0, av0);       // after the last chunk: read and dropped
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      ub_cur = ub_next;
      MIE_STAMP(4 + (c - c_lo));
    }
    // (the epilogue reuses the staging buffers: every read of them that matters was waited for in front of the
    // last barrier; the operand read behind it returns whatever a faster wave has parked there, and is dropped)
  } else {
    for (int c = c_lo; c < c_hi; ++c) {
      const bool more = c + 1 < c_hi;
      const int cn = more ? c + 1 : c;      // after the last chunk: redundant re-load, never stored
      ub_next = chunk_b(cn);
      stage_load(cn);
      const TL* sin = sbuf + ((c - c_lo) % NBUF) * (PL * STAGE);
      // A operands are read one unit ahead as well (two register sets); the scheduling barriers
      // pin "issue the loads for later units, then multiply this unit" so that the compiler can
      // neither sink the prefetches next to their uses nor hoist them all to the top.
      float4 av[2][2][PL];
      load_a(sin, 0, av[0]);
#pragma unroll
      for (int i = 0; i < UPC; ++i) {
        // B operands of the unit PD ahead (the first units of the next chunk at the end)
        if (PD > 0) {
          const int ip = i + PD;
          if (ip < UPC) load_b(ub_cur, ip, bring[ip % RING]);
          else load_b(ub_next, ip - UPC, bring[ip % RING]);
        }
        if (i + 1 < UPC) load_a(sin, i + 1, av[(i + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
        mma(i, av[i & 1], bring[i % RING]);
        __builtin_amdgcn_sched_barrier(0);
        if (PD == 0) load_b(ub_next, 0, bring[0]);   // ring of one: reload right after use
      }
      if (NBUF == 1 && !UP) __syncthreads();   // every wave is done reading the only buffer (UP: stage_store syncs)
      if (more) stage_store((c - c_lo + 1) % NBUF);
      __syncthreads();
      ub_cur = ub_next;
      MIE_STAMP(4 + (c - c_lo));
    }
  }

  // ---- epilogue -----------------------------------------------------------------------------------
  // acc[mb][nb][r] of this lane is output pixel p = 32*mb + 8*(r/4) + 4*half + r%4,
  // channel column wn*32*NB + 32*nb + lane%32 of the workgroup's slab.
  if constexpr (X3) {
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mb][nb][r] += accs[mb][nb][r];
  }
  if constexpr (GATES) {
    // ConvLSTM gate chain as the epilogue.  The filter columns are interleaved by gate: column 4*hc + g is
    // gate g (in, remember, out, cell) of hidden channel hc, so a workgroup owns all four gates of its
    // CO_BLK/4 hidden channels.  Every wave parks its accumulators in LDS; a thread then sums the k-split
    // partials of the four gate columns of one (pixel, hidden channel) and runs the chain on the reservoirs.
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
    // An item is one pixel x four adjacent hidden channels: their 16 gate columns are four 16-byte groups in LDS
    // and 64 contiguous bytes of the gate reservoir, their cell / previous-cell reservoirs one 16-byte group each,
    // their state deltas 16 (fp32) or 8 (bf16) bytes.
    constexpr int HC = CO_BLK / 4;             // hidden channels of this workgroup
    constexpr int HG = HC / 4;                 // groups of four of them
    constexpr int NIT = 64 * HG;               // items of the tile
    constexpr int PERG = (NIT + 255) / 256;    // items per thread (the 32-column slab has 128 items: half the threads idle)
    const int hid = a.hid;
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < PERG; ++i) {
      const int idx = tid + 256 * i;
      if (idx >= NIT) continue;
      const int p = idx / HG, g4 = idx - p * HG;
      const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
      if (oy >= hout || ox >= wout) continue;
      const long long pix = ((long long)n * hout + oy) * wout + ox;
      const long long ho = pix * hid + co0 / 4 + 4 * g4;
      if (!a.ts.pixmask[pix]) {               // inactive pixel of an active tile: clean zeros
        mie_st4(a.g_dh, ho, zero4);
        mie_st4(a.g_dc, ho, zero4);
        continue;
      }
      float4 dg[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        dg[j] = *reinterpret_cast<const float4*>(&smem[p * CO_BLK + 16 * g4 + 4 * j]);
#pragma unroll
        for (int k2 = 1; k2 < WK; ++k2) {
          const float4 part = *reinterpret_cast<const float4*>(&smem[k2 * (64 * CO_BLK) + p * CO_BLK + 16 * g4 + 4 * j]);
          dg[j].x += part.x; dg[j].y += part.y; dg[j].z += part.z; dg[j].w += part.w;
        }
      }
      conv_gates_item<T>(a, pix, ho, pix * a.cout + co0 + 16 * g4, dg);
    }
  } else {
    // the last barrier of the main loop has retired every read of the staging buffers that is used
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
#pragma unroll
    for (int h0 = 0; h0 < PER; h0 += PB) {       // the 128-column slabs in two passes of four groups per thread
      if (!EARLY || SPLIT) epilogue_fetch(h0);
      float4 v[PB];
#pragma unroll
      for (int i = 0; i < PB; ++i) {
        const int idx = tid + 256 * (h0 + i);      // group idx: pixel idx / QPP, channels 4 * (idx % QPP) ...
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
        for (int i = 0; i < PB; ++i)
          if (e_ok[i]) *reinterpret_cast<float4*>(plane + e_off[i]) = v[i];
      } else {
        conv_epilogue_store4<T, PB>(a, e_off, e_co, e_ok, v, e_r0, e_add, e_live);
      }
    }
  }
  MIE_STAMP(14);
}

// Second half of a SPLIT launch: per active tile the `parts` partial planes are added in order and
// the ordinary epilogue (addend, reservoir, activation) runs; stale tiles are zeroed.  One thread per
// (pixel, channel), channels fastest.
template <typename T>
__global__ __launch_bounds__(256) void k_conv_split_finish(ConvArgsT<T> a, int parts) {
  int n, y0, x0;
  const int tk = mie_pick_tile(a.ts, blockIdx.x + conv_args_entry_zero(a), n, y0, x0);
  if (tk == 0) return;
  const int hout = a.ts.h, wout = a.ts.w, cout = a.cout;
  const int cb = (((cout + (int)gridDim.y - 1) / (int)gridDim.y) + 3) & ~3;      // channels of this block (whole groups of four)
  const int c0 = (int)blockIdx.y * cb;
  const int cn = (cout - c0 < cb) ? cout - c0 : cb;
  const int qn = cn >> 2;                                             // groups of four adjacent channels
  for (int idx = threadIdx.x; idx < 64 * qn; idx += 256) {
    const int p = idx / qn, co = c0 + 4 * (idx - p * qn);
    const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
    if (oy >= hout || ox >= wout) continue;
    const long long off = (((long long)n * hout + oy) * wout + ox) * cout + co;
    if (tk == 2) {
      mie_st4(a.out, off, make_float4(0.f, 0.f, 0.f, 0.f));
      continue;
    }
    float4 sum = *reinterpret_cast<const float4*>(a.ws + off);
    for (int q = 1; q < parts; ++q) {
      const float4 part = *reinterpret_cast<const float4*>(a.ws + (long long)q * a.ws_plane + off);
      sum.x += part.x; sum.y += part.y; sum.z += part.z; sum.w += part.w;
    }
    const long long offs[1] = {off};
    const int cos[1] = {co};
    const bool oks[1] = {true};
    const float4 accs[1] = {sum};
    float4 r0[1], add[1];
    conv_epilogue_load4<T, 1>(a, offs, oks, r0, add);
    conv_epilogue_store4<T, 1>(a, offs, cos, oks, accs, r0, add);
  }
}

// Second half of a split gates conv: per active tile the partial planes of the 4 * hid gate columns are added in
// order and the ConvLSTM gate chain runs on the sums; stale tiles get zero state deltas.  One thread per (pixel, four
// adjacent hidden channels), blockIdx.y over groups of hidden channels.
template <typename T>
__global__ __launch_bounds__(256) void k_gates_split_finish(ConvArgsT<T> a, int parts) {
  int n, y0, x0;
  const int tk = mie_pick_tile(a.ts, blockIdx.x + conv_args_entry_zero(a), n, y0, x0);
  if (tk == 0) return;
  const int hout = a.ts.h, wout = a.ts.w, hid = a.hid;
  const int hg_all = hid / 4;                                         // groups of four hidden channels
  const int hgb = (hg_all + (int)gridDim.y - 1) / (int)gridDim.y;      // groups of this block
  const int g_lo = (int)blockIdx.y * hgb;
  const int gn = (hg_all - g_lo < hgb) ? hg_all - g_lo : hgb;
  const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int idx = threadIdx.x; idx < 64 * gn; idx += 256) {
    const int p = idx / gn, g4 = g_lo + (idx - p * gn);
    const int oy = y0 + (p >> 3), ox = x0 + (p & 7);
    if (oy >= hout || ox >= wout) continue;
    const long long pix = ((long long)n * hout + oy) * wout + ox;
    const long long ho = pix * hid + 4 * g4;
    if (tk == 2 || !a.ts.pixmask[pix]) {
      mie_st4(a.g_dh, ho, zero4);
      mie_st4(a.g_dc, ho, zero4);
      continue;
    }
    const long long go = pix * a.cout + 16 * g4;
    float4 dg[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      dg[j] = *reinterpret_cast<const float4*>(a.ws + go + 4 * j);
      for (int q = 1; q < parts; ++q) {
        const float4 part = *reinterpret_cast<const float4*>(a.ws + (long long)q * a.ws_plane + go + 4 * j);
        dg[j].x += part.x; dg[j].y += part.y; dg[j].z += part.z; dg[j].w += part.w;
      }
    }
    conv_gates_item<T>(a, pix, ho, go, dg);
  }
}

// A launch is split when it has at most 128 workgroups, at least 4 staged chunks and a workspace:
// into the largest power of two of parts (up to 8) that keeps the launch at 256 workgroups or fewer (one
// per CU: measured on MI355X, a second workgroup per CU costs more in per-workgroup set-up than it gains),
// leaves every part a chunk, and fits the workspace.  Returns false when the launch is not split.
// Number of parts (0: the launch is not split) for `groups` (tile, slab) pairs of `nch` staged chunks each; sets the
// plane size of the workspace.
template <typename T>
int split_parts(ConvArgsT<T>& a, long long groups, int nch) {
  static const int max_groups = [] { const char* e = getenv("MIE_CONV_SPLIT_GROUPS"); return e ? atoi(e) : 128; }();
  static const int max_wgs = [] { const char* e = getenv("MIE_CONV_SPLIT_WGS"); return e ? atoi(e) : 256; }();
  static const int most = [] {      // MIE_CONV_SPLIT caps the number of parts (1: never split): a tuning knob, read once
    const char* e = getenv("MIE_CONV_SPLIT");
    return e ? atoi(e) : 8;
  }();
  if (a.ws == nullptr || groups > max_groups || nch < 4) return 0;
  a.xcd_fs = 0;
  a.ws_plane = (long long)a.ts.n * a.ts.h * a.ts.w * a.cout;
  int parts = 1;
  while (2 * parts <= most && 2 * parts <= nch && groups * (2 * parts) <= max_wgs && (long long)(2 * parts) * a.ws_plane <= a.ws_floats)
    parts *= 2;
  return parts < 2 ? 0 : parts;
}

template <typename T>
void launch_split_finish(const ConvArgsT<T>& a, unsigned cap, int parts, hipStream_t st) {
  unsigned ny = (unsigned)((1024 + cap - 1) / cap);
  if (ny > (unsigned)(a.cout / 4)) ny = (unsigned)(a.cout / 4);
  if (ny < 1) ny = 1;
  hipLaunchKernelGGL(k_conv_split_finish<T>, dim3(cap, ny), dim3(256), 0, st, a, parts);
}

template <typename T, int K, int S>
bool launch_split(const ConvArgsT<T>& a0, unsigned cap, hipStream_t st) {
  constexpr int CC = stage_channels(K, S, false) * (4 / (int)sizeof(T));
  if (a0.ws == nullptr || a0.refresh || a0.cout % 32 != 0 || a0.c1 % CC != 0 || a0.c2 % CC != 0) return false;
  ConvArgsT<T> a = a0;
  const int parts = split_parts(a, (long long)cap * (a0.cout / 32), (a0.c1 + a0.c2) / CC);
  if (parts == 0) return false;
  bool x3 = false;
  if constexpr (sizeof(T) == 4 && S == 1 && (K == 3 || K == 5)) x3 = a.x3 != 0;
  if (x3) {
    if constexpr (sizeof(T) == 4 && S == 1 && (K == 3 || K == 5))
      hipLaunchKernelGGL((k_conv_mfma<T, K, S, 1, 1, false, false, false, true, true>), dim3(cap, a.cout / 32, parts), dim3(256), 0, st, a);
  } else {
    hipLaunchKernelGGL((k_conv_mfma<T, K, S, 1, 1, false, false, false, true>), dim3(cap, a.cout / 32, parts), dim3(256), 0, st, a);
  }
  launch_split_finish(a, cap, parts, st);
  return true;
}

// The split form of the 5x5 conv over up2x(x + x2): the chunks of the (summed) input split as above, the plain finish.
template <typename T>
bool launch_up_split(const ConvArgsT<T>& a0, unsigned cap, hipStream_t st) {
  constexpr int CC = stage_channels(5, 1, false) * (4 / (int)sizeof(T));
  static const bool on = [] { const char* e = getenv("MIE_CONV_SPLIT_UP"); return e == nullptr || atoi(e) != 0; }();   // tuning knob
  if (!on || a0.ws == nullptr || a0.cout % 32 != 0 || a0.c1 % CC != 0) return false;
  ConvArgsT<T> a = a0;
  const int parts = split_parts(a, (long long)cap * (a0.cout / 32), a0.c1 / CC);
  if (parts == 0) return false;
  bool x3 = false;
  if constexpr (sizeof(T) == 4) x3 = a.x3 != 0;
  if (x3) {
    if constexpr (sizeof(T) == 4)
      hipLaunchKernelGGL((k_conv_mfma<T, 5, 1, 1, 1, false, false, true, true, true>), dim3(cap, a.cout / 32, parts), dim3(256), 0, st, a);
  } else {
    hipLaunchKernelGGL((k_conv_mfma<T, 5, 1, 1, 1, false, false, true, true>), dim3(cap, a.cout / 32, parts), dim3(256), 0, st, a);
  }
  launch_split_finish(a, cap, parts, st);
  return true;
}

// The split form of a ConvLSTM's gates conv: the contraction as a plain split 3x3 conv of the two inputs (the partial
// sums of all 4 * hid gate columns go to the workspace), then the gate chain in the finish kernel.
template <typename T>
bool launch_gates_split(const ConvArgsT<T>& a0, unsigned cap, hipStream_t st) {
  constexpr int CC = stage_channels(3, 1, false) * (4 / (int)sizeof(T));
  static const bool on = [] { const char* e = getenv("MIE_CONV_SPLIT_GATES"); return e == nullptr || atoi(e) != 0; }();   // tuning knob
  if (!on || a0.ws == nullptr || a0.cout != 4 * a0.hid || a0.hid % 8 != 0 || a0.c1 % CC != 0 || a0.c2 % CC != 0) return false;
  ConvArgsT<T> a = a0;
  const int parts = split_parts(a, (long long)cap * (a0.cout / 32), (a0.c1 + a0.c2) / CC);
  // (two parts do not pay for the second launch: E2Depth-incr 128x128 frame 0.2685 -> 0.2699 ms, measured; four do)
  if (parts < 4) return false;
  bool x3 = false;
  if constexpr (sizeof(T) == 4) x3 = a.x3 != 0;
  if (x3) {
    if constexpr (sizeof(T) == 4)
      hipLaunchKernelGGL((k_conv_mfma<T, 3, 1, 1, 1, false, false, false, true, true>), dim3(cap, a.cout / 32, parts), dim3(256), 0, st, a);
  } else {
    hipLaunchKernelGGL((k_conv_mfma<T, 3, 1, 1, 1, false, false, false, true>), dim3(cap, a.cout / 32, parts), dim3(256), 0, st, a);
  }
  unsigned ny = (unsigned)((1024 + cap - 1) / cap);
  if (ny > (unsigned)(a.hid / 4)) ny = (unsigned)(a.hid / 4);
  if (ny < 1) ny = 1;
  hipLaunchKernelGGL(k_gates_split_finish<T>, dim3(cap, ny), dim3(256), 0, st, a, parts);
  return true;
}

// Output channels per workgroup (the slab 32*NB*WN) for a launch of `cap` tiles: the widest of
// 128 / 64 / 32 that still gives the chip at least 400 workgroups when every tile is active
// (256 CUs, up to 3 workgroups resident on each), else the narrowest the staging depth of this
// (K, S) allows.  Measured on MI355X over the layer shapes of both network sizes: wider slabs
// re-read less of the input tile but leave CUs idle on the small planes; the 256-wide variant
// (two 32-column blocks per wave) lost to the 128-wide one on every shape and is only taken
// when forced.  The environment
// variable MIE_CONV_SLAB (32, 64, 128 or 256) overrides the choice where the shape allows it --
// a tuning knob for measurements, read once.
int forced_slab() {
  static const int v = [] {
    const char* e = getenv("MIE_CONV_SLAB");
    return e ? atoi(e) : 0;
  }();
  return v;
}

template <int K, int S, bool HALF>
int pick_slab(int cout, unsigned cap) {
  constexpr int NQ = stage_channels(K, S, HALF) / 8;
  const bool ok128 = cout % 128 == 0, ok64 = NQ >= 2 && cout % 64 == 0;
  const bool ok32 = NQ >= 4 && cout % 32 == 0;
  const int f = forced_slab();
  if ((f == 128 && ok128) || (f == 64 && ok64) || (f == 32 && ok32)) return f;
  const long long want = 400;
  if (ok128 && ((long long)cap * (cout / 128) >= want || (!ok64 && !ok32))) return 128;
  if (ok64 && ((long long)cap * (cout / 64) >= want || !ok32)) return 64;
  if (ok32) return 32;
  return 0;
}

// XCD-aware launch order (see the kernel): chooses the number of slab groups a.xcd_fs in {1, 2, 4, 8}
// (a divisor of the slab count) that minimises what the 8 L2s fetch in total -- the filter 8 / xcd_fs
// times plus the input xcd_fs times -- and returns the grid's x extent: the tile capacity rounded up to a
// multiple of 8, plus 16 (the shares of active and of stale work are rounded up separately).  The
// environment variable MIE_CONV_XCD forces the number of groups (0: plain launch order, a.xcd_fs = 0) --
// a tuning knob for measurements, read once.
template <typename T>
unsigned xcd_plan(ConvArgsT<T>& a, unsigned cap, int nslabs, int k, bool up = false) {
  static const int forced = [] {
    const char* e = getenv("MIE_CONV_XCD");
    return e ? atoi(e) : -1;
  }();
  a.xcd_fs = 0;
  if (forced == 0) return cap;
  const double cin = (double)a.c1 + a.c2;
  const double filt = cin * k * k * a.cout;
  const double in = (double)a.ts.n * a.h_in * a.w_in * (up ? 0.5 * a.c1 : cin);
  int best = 1;
  double cost = 8 * filt + in;
  for (int fs = 2; fs <= 8; fs *= 2) {
    if (nslabs % fs != 0) break;
    const double c = (8 / fs) * filt + fs * in;
    if (c < cost) cost = c, best = fs;
  }
  if (forced > 0 && 8 % forced == 0 && nslabs % forced == 0) best = forced;
  a.xcd_fs = best;
  return ((cap + 7u) & ~7u) + 16u;
}

// X3 kernels (fp32 deltas, a.x3 set, the filter copy in the three-term layout): 3x3 / 5x5, stride 1, input channels in
// whole chunks of 32, output slabs of 128 / 64 / 32 columns by the same rule as above.
// Stride 1 first looks for the widest slab that makes the launch one round of more than half a chip of workgroups
// (129 .. 256): measured on MI355X, one workgroup per CU with twice the columns beats one and a half rounds of the
// narrow ones (5x5 256->128 at 66x88: 198 workgroups of 64 columns 61-65 us, 396 of 32 columns 71-74 us; 3x3 gates conv
// 256+256->1024 at 33x44: 240 of 128 columns 53 us, 480 of 64 columns 57 us); at stride 2, whose workgroups are short,
// it does not (28 vs 29 us).
inline int pick_slab_x3(int cout, unsigned cap, int s) {
  const bool ok128 = cout % 128 == 0, ok64 = cout % 64 == 0, ok32 = cout % 32 == 0;
  const int f = forced_slab();
  if ((f == 128 && ok128) || (f == 64 && ok64) || (f == 32 && ok32)) return f;
  if (s == 1) {
    const int widths[3] = {128, 64, 32};
    const bool oks[3] = {ok128, ok64, ok32};
    for (int i = 0; i < 3; ++i) {
      const long long wgs = (long long)cap * (cout / widths[i]);
      if (oks[i] && wgs > 128 && wgs <= 256) return widths[i];
    }
  }
  const long long want = 400;
  if (ok128 && ((long long)cap * (cout / 128) >= want || (!ok64 && !ok32))) return 128;
  if (ok64 && ((long long)cap * (cout / 64) >= want || !ok32)) return 64;
  if (ok32) return 32;
  return 0;
}
inline bool x3_takes(int k, int s, int c1, int c2, int cout) {
  // (3x3 stride 2 was measured too: no faster than the fp32 instruction, 15-29 us either way, and it has a split form)
  if (s == 2) return k == 5 && c1 % 16 == 0 && c2 % 16 == 0 && cout % 32 == 0;
  return (k == 3 || k == 5) && s == 1 && c1 % 32 == 0 && c2 % 32 == 0 && cout % 32 == 0;
}

template <int K, bool GATES, bool UP, int S = 1>
bool launch_x3(const ConvArgsT<float>& a0, unsigned cap, hipStream_t st) {
  ConvArgsT<float> a = a0;
  const int cout = a.cout;
  if (!x3_takes(K, S, a.c1, UP ? 0 : a.c2, cout)) return false;
  switch (pick_slab_x3(cout, cap, S)) {
    case 128:
      hipLaunchKernelGGL((k_conv_mfma<float, K, S, 4, 1, false, GATES, UP, false, true>), dim3(xcd_plan(a, cap, cout / 128, K, UP), cout / 128), dim3(256), 0, st, a);
      return true;
    case 64:
      hipLaunchKernelGGL((k_conv_mfma<float, K, S, 2, 1, false, GATES, UP, false, true>), dim3(xcd_plan(a, cap, cout / 64, K, UP), cout / 64), dim3(256), 0, st, a);
      return true;
    case 32:
      hipLaunchKernelGGL((k_conv_mfma<float, K, S, 1, 1, false, GATES, UP, false, true>), dim3(xcd_plan(a, cap, cout / 32, K, UP), cout / 32), dim3(256), 0, st, a);
      return true;
    default:
      return false;
  }
}

template <typename T, int K, int S, bool HALF>
bool launch_depth(const ConvArgsT<T>& a0, unsigned cap, hipStream_t st) {
  constexpr int NQ = stage_channels(K, S, HALF) / 8;
  ConvArgsT<T> a = a0;
  const int cout = a.cout;
  switch (pick_slab<K, S, HALF>(cout, cap)) {
    case 128:
      hipLaunchKernelGGL((k_conv_mfma<T, K, S, 4, 1, HALF>), dim3(xcd_plan(a, cap, cout / 128, K), cout / 128), dim3(256), 0, st, a);
      return true;
    case 64:
      if constexpr (NQ >= 2) {
        hipLaunchKernelGGL((k_conv_mfma<T, K, S, 2, 1, HALF>), dim3(xcd_plan(a, cap, cout / 64, K), cout / 64), dim3(256), 0, st, a);
        return true;
      }
      return false;
    case 32:
      if constexpr (NQ >= 4) {
        hipLaunchKernelGGL((k_conv_mfma<T, K, S, 1, 1, HALF>), dim3(xcd_plan(a, cap, cout / 32, K), cout / 32), dim3(256), 0, st, a);
        return true;
      }
      return false;
    default:
      return false;
  }
}

// The 5x5 stride-1 conv over up2x(x + x2): full staging depth only.
template <typename T>
bool launch_up(const ConvArgsT<T>& a0, unsigned cap, hipStream_t st) {
  if (launch_up_split<T>(a0, cap, st)) return true;
  if constexpr (sizeof(T) == 4) {
    if (a0.x3) return launch_x3<5, false, true>(a0, cap, st);
  }
  constexpr int FULL = stage_channels(5, 1) * (4 / (int)sizeof(T));
  if (a0.c1 % FULL != 0) return false;
  ConvArgsT<T> a = a0;
  const int cout = a.cout;
  switch (pick_slab<5, 1, false>(cout, cap)) {
    case 128:
      hipLaunchKernelGGL((k_conv_mfma<T, 5, 1, 4, 1, false, false, true>), dim3(xcd_plan(a, cap, cout / 128, 5, true), cout / 128), dim3(256), 0, st, a);
      return true;
    case 64:
      hipLaunchKernelGGL((k_conv_mfma<T, 5, 1, 2, 1, false, false, true>), dim3(xcd_plan(a, cap, cout / 64, 5, true), cout / 64), dim3(256), 0, st, a);
      return true;
    case 32:
      hipLaunchKernelGGL((k_conv_mfma<T, 5, 1, 1, 1, false, false, true>), dim3(xcd_plan(a, cap, cout / 32, 5, true), cout / 32), dim3(256), 0, st, a);
      return true;
    default:
      return false;
  }
}

// The gates conv of a ConvLSTM: 3x3, stride 1, full staging depth, gate chain in the epilogue.
template <typename T>
bool launch_gates(const ConvArgsT<T>& a0, unsigned cap, hipStream_t st) {
  if (launch_gates_split<T>(a0, cap, st)) return true;
  if constexpr (sizeof(T) == 4) {
    if (a0.x3) return a0.cout == 4 * a0.hid && a0.hid % 8 == 0 && launch_x3<3, true, false>(a0, cap, st);
  }
  constexpr int FULL = stage_channels(3, 1) * (4 / (int)sizeof(T));
  if (a0.c1 % FULL != 0 || a0.c2 % FULL != 0 || a0.cout != 4 * a0.hid || a0.hid % 8 != 0) return false;
  ConvArgsT<T> a = a0;
  const int cout = a.cout;
  switch (pick_slab<3, 1, false>(cout, cap)) {
    case 128:
      hipLaunchKernelGGL((k_conv_mfma<T, 3, 1, 4, 1, false, true>), dim3(xcd_plan(a, cap, cout / 128, 3), cout / 128), dim3(256), 0, st, a);
      return true;
    case 64:
      hipLaunchKernelGGL((k_conv_mfma<T, 3, 1, 2, 1, false, true>), dim3(xcd_plan(a, cap, cout / 64, 3), cout / 64), dim3(256), 0, st, a);
      return true;
    case 32:
      hipLaunchKernelGGL((k_conv_mfma<T, 3, 1, 1, 1, false, true>), dim3(xcd_plan(a, cap, cout / 32, 3), cout / 32), dim3(256), 0, st, a);
      return true;
    default:
      return false;
  }
}

// Staging depth: the full one when both inputs' channel counts are multiples of it, else
// (stride 2 only) the half one.
template <typename T, int K, int S>
bool launch_ks(const ConvArgsT<T>& a, unsigned cap, hipStream_t st) {
  constexpr int MULT = 4 / (int)sizeof(T);
  constexpr int FULL = stage_channels(K, S) * MULT;
  if (a.c1 % FULL == 0 && a.c2 % FULL == 0 && pick_slab<K, S, false>(a.cout, cap) != 0)
    return launch_depth<T, K, S, false>(a, cap, st);
  if constexpr (S == 2) {
    constexpr int HALFC = stage_channels(K, S, true) * MULT;
    if (a.c1 % HALFC == 0 && a.c2 % HALFC == 0) return launch_depth<T, K, S, true>(a, cap, st);
  }
  return false;
}

}  // namespace

namespace {
template <typename T>
bool launch_any(const ConvArgsT<T>& a, int k, int s, unsigned cap, hipStream_t st) {
  if constexpr (sizeof(T) == 4) {
    if (a.x3) {
      if (k == 3 && s == 1) return launch_split<T, 3, 1>(a, cap, st) || launch_x3<3, false, false>(a, cap, st);
      if (k == 5 && s == 1) return launch_split<T, 5, 1>(a, cap, st) || launch_x3<5, false, false>(a, cap, st);
      if (k == 5 && s == 2) return launch_x3<5, false, false, 2>(a, cap, st);     // (no split form at stride 2)
      return false;
    }
  }
  switch (k * 10 + s) {
    case 11: return launch_ks<T, 1, 1>(a, cap, st);
    case 12: return launch_ks<T, 1, 2>(a, cap, st);
    case 31: return launch_split<T, 3, 1>(a, cap, st) || launch_ks<T, 3, 1>(a, cap, st);
    case 32: return launch_split<T, 3, 2>(a, cap, st) || launch_ks<T, 3, 2>(a, cap, st);
    case 51: return launch_split<T, 5, 1>(a, cap, st) || launch_ks<T, 5, 1>(a, cap, st);
    case 52: return launch_split<T, 5, 2>(a, cap, st) || launch_ks<T, 5, 2>(a, cap, st);
    case 71: return launch_ks<T, 7, 1>(a, cap, st);
    case 72: return launch_ks<T, 7, 2>(a, cap, st);
    default: return false;
  }
}
}  // namespace

