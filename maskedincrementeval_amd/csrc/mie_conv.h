// Arguments shared by the masked-conv kernels (VALU paths in mie_conv.hip, matrix-core
// path in mie_conv_mfma_impl.h).
#pragma once
#include "mie_common.h"

// T = element type of the deltas (inputs, output, addend) and of the matrix-core filter copy:
// float or mie_bf16.  Reservoirs, bias, the plain filter and all accumulation are fp32.
template <typename T>
struct ConvArgsT {
  const T* x; const uint8_t* xm; int c1;
  const T* x2; const uint8_t* x2m; int c2;
  int h_in, w_in;
  const float* filt; int cin_total;
  const T* filt_mc;                 // matrix-core copy of the filter (mie_pack_filter) or NULL
  int pad, cout;
  T* out; float* res; int act; float slope;
  const T* addend;                  // optional delta added to the conv result before the epilogue
  int refresh; const float* bias;   // dense refresh: out = act(acc + bias), res = acc + bias
  // ConvLSTM gate chain fused into the epilogue (matrix-core path, GATES kernels): `res` is the gate
  // pre-activation reservoir in the conv's column order, `out` is unused; the rest as in
  // mie_convlstm_gates_incr.
  int hid;
  const T* g_cpd; const uint8_t* g_cpm; float* g_cpres; float* g_cres; T* g_dh; T* g_dc;
  // Workspace of the matrix-core path for launches of very few tiles (SPLIT kernels): fp32 partial sums,
  // one plane of n*h*w*cout floats per part.  NULL: such launches are not split.
  float* ws; long long ws_floats; long long ws_plane;
  // Matrix-core path: launch order permuted per XCD (number of slab groups, 0 = plain order); set by the launchers.
  int xcd_fs;
  // Matrix-core path, fp32 deltas: filt_mc is the three-term bf16 copy and the contraction runs as six bf16 products
  // per term pair (MIE_DTYPE_F32_BF16X3).
  int x3;
  TileSetDev ts;
};
typedef ConvArgsT<float> ConvArgs;

// The argument block is five cache lines of device memory that no cache holds when a launch starts.  Left to itself the
// compiler fetches a field where it is first used, and a workgroup then stalls on those lines one after the other on its
// way to its first loads.  This reads one field of every line in one batch at the kernel's entry, so that the later
// reads hit the scalar cache, and returns zero -- out of an instruction the compiler cannot see through, to be added to
// the workgroup index, so that the reads can neither be dropped nor moved down.  (The asm is not volatile, which would
// turn every later uniform load into a vector load.)  Measured on the 264x352 frame: 0.565 -> 0.562 ms.
template <typename T>
static __device__ __forceinline__ int conv_args_entry_zero(const ConvArgsT<T>& a) {
  const int touch = a.c1 ^ a.cout ^ a.hid ^ a.xcd_fs ^ a.ts.n;      // (the fifth line holds the list pointers, read next)
  int zero;
  asm("s_and_b32 %0, %1, 0" : "=s"(zero) : "s"(touch) : "scc");
  return zero;
}

// Epilogue for one output element (linear offset off, output channel co).
template <typename T>
static __device__ __forceinline__ void conv_store(const ConvArgsT<T>& a, long long off, int co, float acc) {
  if (a.addend) acc += mie_ld(a.addend, off);
  if (a.refresh) {
    const float v = a.bias ? acc + a.bias[co] : acc;
    if (a.res) a.res[off] = v;
    mie_st(a.out, off, mie_act(a.act, a.slope, v));
  } else if (a.res) {
    const float r0 = a.res[off], r1 = r0 + acc;
    a.res[off] = r1;
    mie_st(a.out, off, mie_act(a.act, a.slope, r1) - mie_act(a.act, a.slope, r0));
  } else {
    mie_st(a.out, off, acc);
  }
}

// The same epilogue for N elements of one thread, in two halves.  conv_epilogue_load issues every
// reservoir / addend load of the thread as one batch; a kernel calls it long before the values are
// needed (at its very start: an output element belongs to one thread of one workgroup, nobody else
// touches its reservoir), so their latency hides behind the contraction.  conv_epilogue_store adds
// the accumulators and writes.  Elements with ok[i] == false are skipped.
template <typename T, int N>
static __device__ __forceinline__ void conv_epilogue_load(const ConvArgsT<T>& a, const long long (&off)[N],
                                                          const bool (&ok)[N], float (&r0)[N],
                                                          float (&add)[N]) {
  const bool want_res = a.res != nullptr && !a.refresh;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    r0[i] = 0.f;
    add[i] = 0.f;
    if (ok[i]) {
      if (a.addend) add[i] = mie_ld(a.addend, off[i]);
      if (want_res) r0[i] = a.res[off[i]];
    }
  }
}

template <typename T, int N>
static __device__ __forceinline__ void conv_epilogue_store(const ConvArgsT<T>& a, const long long (&off)[N],
                                                           const int (&co)[N], const bool (&ok)[N],
                                                           const float (&acc)[N], const float (&r0)[N],
                                                           const float (&add)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) {
    if (!ok[i]) continue;
    float v = acc[i] + add[i];
    if (a.refresh) {
      if (a.bias) v += a.bias[co[i]];
      if (a.res) a.res[off[i]] = v;
      mie_st(a.out, off[i], mie_act(a.act, a.slope, v));
    } else if (a.res) {
      const float r1 = r0[i] + v;
      a.res[off[i]] = r1;
      mie_st(a.out, off[i], mie_act(a.act, a.slope, r1) - mie_act(a.act, a.slope, r0[i]));
    } else {
      mie_st(a.out, off[i], v);
    }
  }
}

// The same for N groups of four adjacent output channels of one pixel each (off[i] = offset of the first of
// the four, a multiple of 4; co[i] its channel): 16-byte reservoir accesses, 16- / 8-byte delta accesses.
// Pixels of an active tile that lie outside the output pixel mask (live[i] false; the mask covers every pixel whose
// window holds an active input pixel, so acc and addend are exactly zero there) keep their reservoir untouched -- r1 =
// r0 + 0 would store the value just read -- and get a zero delta: conv_epilogue_load4 fetches nothing for them
// (pass live as its ok), conv_epilogue_store4 writes the zeros.  A dense refresh treats every pixel as live.
template <typename T, int N>
static __device__ __forceinline__ void conv_epilogue_load4(const ConvArgsT<T>& a, const long long (&off)[N],
                                                           const bool (&ok)[N], float4 (&r0)[N], float4 (&add)[N]) {
  const bool want_res = a.res != nullptr && !a.refresh;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    r0[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    add[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (ok[i]) {
      if (a.addend) add[i] = mie_ld4(a.addend, off[i]);
      if (want_res) r0[i] = mie_ld4(a.res, off[i]);
    }
  }
}

template <typename T, int N>
static __device__ __forceinline__ void conv_epilogue_store4(const ConvArgsT<T>& a, const long long (&off)[N],
                                                            const int (&co)[N], const bool (&ok)[N],
                                                            const float4 (&acc)[N], const float4 (&r0)[N],
                                                            const float4 (&add)[N], const bool (&live)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) {
    if (!ok[i]) continue;
    if (!live[i]) {
      mie_st4(a.out, off[i], make_float4(0.f, 0.f, 0.f, 0.f));
      continue;
    }
    float4 v = make_float4(acc[i].x + add[i].x, acc[i].y + add[i].y, acc[i].z + add[i].z, acc[i].w + add[i].w);
    if (a.refresh) {
      if (a.bias) {
        v.x += a.bias[co[i]]; v.y += a.bias[co[i] + 1]; v.z += a.bias[co[i] + 2]; v.w += a.bias[co[i] + 3];
      }
      if (a.res) mie_st4(a.res, off[i], v);
      mie_st4(a.out, off[i], make_float4(mie_act(a.act, a.slope, v.x), mie_act(a.act, a.slope, v.y),
                                         mie_act(a.act, a.slope, v.z), mie_act(a.act, a.slope, v.w)));
    } else if (a.res) {
      const float4 r1 = make_float4(r0[i].x + v.x, r0[i].y + v.y, r0[i].z + v.z, r0[i].w + v.w);
      mie_st4(a.res, off[i], r1);
      mie_st4(a.out, off[i],
              make_float4(mie_act(a.act, a.slope, r1.x) - mie_act(a.act, a.slope, r0[i].x),
                          mie_act(a.act, a.slope, r1.y) - mie_act(a.act, a.slope, r0[i].y),
                          mie_act(a.act, a.slope, r1.z) - mie_act(a.act, a.slope, r0[i].z),
                          mie_act(a.act, a.slope, r1.w) - mie_act(a.act, a.slope, r0[i].w)));
    } else {
      mie_st4(a.out, off[i], v);
    }
  }
}

template <typename T, int N>
static __device__ __forceinline__ void conv_epilogue_store4(const ConvArgsT<T>& a, const long long (&off)[N],
                                                            const int (&co)[N], const bool (&ok)[N],
                                                            const float4 (&acc)[N], const float4 (&r0)[N],
                                                            const float4 (&add)[N]) {
  conv_epilogue_store4<T, N>(a, off, co, ok, acc, r0, add, ok);
}

template <typename T, int N>
static __device__ __forceinline__ void conv_store_batch(const ConvArgsT<T>& a, const long long (&off)[N],
                                                        const int (&co)[N], const bool (&ok)[N],
                                                        float (&acc)[N]) {
  float r0[N], add[N];
  conv_epilogue_load<T, N>(a, off, ok, r0, add);
  conv_epilogue_store<T, N>(a, off, co, ok, acc, r0, add);
}

// Launches the matrix-core path for kernel size k (1,3,5,7) and stride s (1,2).  Returns false
// if no kernel variant takes the shape (nothing is launched then); mie_conv_mfma_takes says so
// beforehand.
bool mie_launch_conv_mfma(const ConvArgsT<float>& a, int k, int s, unsigned cap, hipStream_t st);
bool mie_launch_conv_mfma(const ConvArgsT<mie_bf16>& a, int k, int s, unsigned cap, hipStream_t st);
// The 3x3 stride-1 conv of a ConvLSTM with the gate chain as its epilogue (a.hid > 0, a.cout = 4*hid,
// filter columns in the gate-interleaved order of mie_conv_gates_masked).
bool mie_launch_conv_gates_mfma(const ConvArgsT<float>& a, unsigned cap, hipStream_t st);
bool mie_launch_conv_gates_mfma(const ConvArgsT<mie_bf16>& a, unsigned cap, hipStream_t st);
// The 5x5 stride-1 pad-2 conv over up2x(a.x + a.x2) (both at half resolution, a.c1 channels each, a.x2
// optional); a.h_in / a.w_in are the up-sampled size.
bool mie_launch_conv_up_mfma(const ConvArgsT<float>& a, unsigned cap, hipStream_t st);
bool mie_launch_conv_up_mfma(const ConvArgsT<mie_bf16>& a, unsigned cap, hipStream_t st);

// The same for bf16 deltas, 64 -> 32 channels, on planes of many tiles: a persistent kernel (mie_upconv_persist.hip).
// Returns false, launching nothing, for other shapes.
bool mie_launch_upconv_persist(const ConvArgsT<mie_bf16>& a, unsigned cap, hipStream_t st);
// ... with the network's tail fused in: the layer's activation increment is not stored; the 1x1 prediction conv over it
// and over `skip` (32 channels, same resolution), the prediction's reservoir update and its activation increment
// (one channel, pred_out) run in the epilogue.  pred_w: [2][32] fp32 (weights of the layer's output, of skip).
bool mie_launch_upconv_pred_persist(const ConvArgsT<mie_bf16>& a, const mie_bf16* skip, const uint8_t* skip_mask,
                                    const float* pred_w, float* pred_res, mie_bf16* pred_out, int pred_act,
                                    float pred_slope, unsigned cap, hipStream_t st);

// Source rows / columns and weights of output index o of a bilinear x2 up-sampling (align_corners =
// False): src = max(0, o/2 - 0.25), upper index clamped to the last row.
static __device__ __forceinline__ void conv_up2x_coef(int o, int in_size, int& i0, int& i1, float& l0, float& l1) {
  const int j = o >> 1;
  if (o & 1) {
    i0 = j; i1 = (j + 1 < in_size) ? j + 1 : j; l0 = 0.75f; l1 = 0.25f;
  } else if (j == 0) {
    i0 = 0; i1 = (1 < in_size) ? 1 : 0; l0 = 1.f; l1 = 0.f;
  } else {
    i0 = j - 1; i1 = j; l0 = 0.25f; l1 = 0.75f;
  }
}
// One value of the up-sampled tile from its four source values (t00 t01 / t10 t11) with column weights lq0, lq1 and row
// weights lr0, lr1: horizontal first, then vertical, every product and sum rounded where it is written here, so that
// every kernel that forms the tile (per pixel, or rows and columns separately) gets the same bits.
static __device__ __forceinline__ float conv_up2x_h(float lq0, float lq1, float t0, float t1) {
  return __fmaf_rn(lq0, t0, __fmul_rn(lq1, t1));
}
static __device__ __forceinline__ float conv_up2x_v(float lr0, float lr1, float h0, float h1) {
  return __fmaf_rn(lr0, h0, __fmul_rn(lr1, h1));
}
// Matrix-core conv for layers of at most 8 input channels (the network heads), one input, k in {3, 5}, Cout % 32
// == 0 (mie_conv_fewcin.hip).  Returns false, launching nothing, for other shapes.
bool mie_launch_conv_fewcin(const ConvArgsT<float>& a, int k, int s, unsigned cap, hipStream_t st);
bool mie_launch_conv_fewcin(const ConvArgsT<mie_bf16>& a, int k, int s, unsigned cap, hipStream_t st);
// The same over up2x(a.x): a.x / a.xm at half resolution, a.h_in / a.w_in the up-sampled size, stride 1.
bool mie_launch_conv_fewcin_up(const ConvArgsT<float>& a, int k, unsigned cap, hipStream_t st);
bool mie_launch_conv_fewcin_up(const ConvArgsT<mie_bf16>& a, int k, unsigned cap, hipStream_t st);

// One element of the ConvLSTM gate chain: pre-activation gate reservoirs r* and their deltas d*, cached
// previous cell state cp and its delta dP, cached cell state c0.  Updates the reservoirs in place and
// returns the deltas of the hidden and the cell state (the chain sigmoid1..3 / tanh1 -> m1 + m2 -> tanh2
// -> m3 of ConvLSTMIncr.forward, incr_modules/e2depth_incr.py:103-120, product rule on cached operands).
static __device__ __forceinline__ float mie_sigm(float v) { return 1.f / (1.f + expf(-v)); }
// Gate chain: sigmoid and tanh through the hardware exponential (v_exp_f32) and reciprocal (v_rcp_f32), about
// 1e-7 absolute error each -- far inside the 1e-5 the results are held to -- at a third of the instructions
// of expf / tanhf / IEEE division; with ten evaluations per (pixel, hidden channel) the chain was bound by
// them.  The same functions serve the dense refresh, so that refresh and increments see one sigmoid.
static __device__ __forceinline__ float mie_gate_sigm(float v) {
  return __builtin_amdgcn_rcpf(1.f + __expf(-v));
}
static __device__ __forceinline__ float mie_gate_tanh(float v) {
  return 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + __expf(2.f * v));     // exp overflow -> rcp(inf) = 0 -> 1
}
static __device__ __forceinline__ void mie_lstm_gate_chain(float& ri, float& rf, float& ro, float& rg, float di,
                                                           float df, float dO, float dG, float& cp, float dP,
                                                           float& cc, float& dh, float& dc) {
  const float ri1 = ri + di, rf1 = rf + df, ro1 = ro + dO, rg1 = rg + dG;
  const float si0 = mie_gate_sigm(ri), dsi = mie_gate_sigm(ri1) - si0;
  const float sf0 = mie_gate_sigm(rf), dsf = mie_gate_sigm(rf1) - sf0;
  const float so0 = mie_gate_sigm(ro), dso = mie_gate_sigm(ro1) - so0;
  const float tg0 = mie_gate_tanh(rg), dtg = mie_gate_tanh(rg1) - tg0;
  const float m1 = (dtg + tg0) * dsi + si0 * dtg;       // m1(in_gate, cell_gate)
  const float m2 = (dP + cp) * dsf + sf0 * dP;          // m2(remember_gate, prev_c)
  const float dcell = m1 + m2;
  const float c0 = cc, c1 = c0 + dcell;
  const float tc0 = mie_gate_tanh(c0), dtc = mie_gate_tanh(c1) - tc0;
  dh = (dtc + tc0) * dso + so0 * dtc;                   // m3(out_gate, tanh(cell))
  dc = dcell;
  ri = ri1; rf = rf1; ro = ro1; rg = rg1;
  cp += dP;
  cc = c1;
}
bool mie_conv_mfma_takes(int k, int s, int dtype, int c1, int c2, int cout);
// The same for the three-term form of fp32 deltas (MIE_DTYPE_F32_BF16X3).
bool mie_conv_x3_takes(int k, int s, int c1, int c2, int cout);
