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
  TileSetDev ts;
};
typedef ConvArgsT<float> ConvArgs;

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

// The same epilogue for N elements of one thread: every reservoir / addend load is issued before
// the first store, so the loads overlap instead of each waiting for the store before it (the
// buffers carry no restrict qualifiers: a store may alias a later load as far as the compiler
// knows).  Elements with ok[i] == false are skipped.
template <typename T, int N>
static __device__ __forceinline__ void conv_store_batch(const ConvArgsT<T>& a, const long long (&off)[N],
                                                        const int (&co)[N], const bool (&ok)[N],
                                                        float (&acc)[N]) {
  float r0[N];
  const bool want_res = a.res != nullptr && !a.refresh;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    r0[i] = 0.f;
    if (ok[i]) {
      if (a.addend) acc[i] += mie_ld(a.addend, off[i]);
      if (want_res) r0[i] = a.res[off[i]];
      if (a.refresh && a.bias) acc[i] += a.bias[co[i]];
    }
  }
#pragma unroll
  for (int i = 0; i < N; ++i) {
    if (!ok[i]) continue;
    if (a.refresh) {
      if (a.res) a.res[off[i]] = acc[i];
      mie_st(a.out, off[i], mie_act(a.act, a.slope, acc[i]));
    } else if (a.res) {
      const float r1 = r0[i] + acc[i];
      a.res[off[i]] = r1;
      mie_st(a.out, off[i], mie_act(a.act, a.slope, r1) - mie_act(a.act, a.slope, r0[i]));
    } else {
      mie_st(a.out, off[i], acc[i]);
    }
  }
}

// Launches the matrix-core path for kernel size k (1,3,5,7) and stride s (1,2).  Returns false
// if no kernel variant takes the shape (nothing is launched then); mie_conv_mfma_takes says so
// beforehand.
bool mie_launch_conv_mfma(const ConvArgsT<float>& a, int k, int s, unsigned cap, hipStream_t st);
bool mie_launch_conv_mfma(const ConvArgsT<mie_bf16>& a, int k, int s, unsigned cap, hipStream_t st);
bool mie_conv_mfma_takes(int k, int s, int dtype, int c1, int c2, int cout);
