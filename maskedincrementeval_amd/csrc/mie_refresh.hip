// State math of the dense refresh pass (gfx950): what a recurrent cell does after its gate convs
// when the reservoirs are (re)filled.  The convs of a refresh run through the masked-conv kernels with
// every tile active (mie_conv_refresh); these kernels turn the gate pre-activations they leave in
// the reservoirs into the cell's dense state and fill the remaining reservoirs, one thread per
// (pixel, hidden channel), so that a refresh holds no framework kernel and can be captured in a graph.
// All are bandwidth-bound passes over dense [n*h*w, hid] tensors.
#include "mie_common.h"
#include "mie_conv.h"      // mie_sigm

namespace {

// prev_c may be c_out or h_out (the state of the previous refresh fed back): a thread reads its element first.
template <typename T>
__global__ __launch_bounds__(256) void k_convlstm_gates_refresh(
    const float* __restrict__ gates_res, int interleaved, const T* prev_c,
    float* __restrict__ cprev_res, float* __restrict__ cell_res, T* h_out, T* c_out, long long total, int hid) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const long long pix = idx / hid;
  const int hc = (int)(idx - pix * hid);
  // gate columns of this hidden channel: [in | remember | out | cell] x hid, or interleaved by gate
  // (column 4*hc + g <-> gate g of hidden channel hc)
  const int col0 = interleaved ? 4 * hc : hc;
  const int step = interleaved ? 1 : hid;
  const float* g = gates_res + pix * (4LL * hid) + col0;
  const float gi = mie_gate_sigm(g[0]), gf = mie_gate_sigm(g[step]), go = mie_gate_sigm(g[2 * step]);
  const float gg = mie_gate_tanh(g[3 * step]);
  const float cp = prev_c ? mie_ld(prev_c, idx) : 0.f;
  const float cell = gi * gg + gf * cp;
  cprev_res[idx] = cp;
  cell_res[idx] = cell;
  mie_st(h_out, idx, go * mie_gate_tanh(cell));
  mie_st(c_out, idx, cell);
}

// `state` may be `prev` (the state of the previous refresh updated in place): a thread reads its element first.
template <typename T>
__global__ __launch_bounds__(256) void k_convgru_gates_refresh(
    const T* __restrict__ update, const T* __restrict__ cand, const T* prev,
    float* __restrict__ diff_res, float* __restrict__ update_res, T* state, long long total) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const float u = mie_ld(update, idx), p = prev ? mie_ld(prev, idx) : 0.f;
  const float d = mie_ld(cand, idx) - p;
  if (diff_res) diff_res[idx] = d;
  if (update_res) update_res[idx] = u;
  mie_st(state, idx, p + d * u);
}

template <typename T>
__global__ __launch_bounds__(256) void k_mul_dense(const T* a, const T* b, T* out, long long total) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  mie_st(out, idx, mie_ld(a, idx) * mie_ld(b, idx));
}

int check_dense(const char* who, long long n, long long h, long long w, long long c, int dtype, long long* total) {
  MIE_REQUIRE(dtype == MIE_DTYPE_F32 || dtype == MIE_DTYPE_BF16, MIE_ERR_UNSUPPORTED, "%s: unknown delta dtype %d",
              who, dtype);
  MIE_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0, MIE_ERR_INVALID_ARG,
              "%s: sizes must be positive (n=%lld h=%lld w=%lld c=%lld)", who, n, h, w, c);
  *total = n * h * w * c;
  MIE_REQUIRE(n * h * w < 0x7fffffffLL && *total < (1LL << 40) && (*total + 255) / 256 < 0x7fffffffLL,
              MIE_ERR_CAPACITY, "%s: tensor too large", who);
  return MIE_OK;
}

}  // namespace

extern "C" int mie_convlstm_gates_refresh(const float* gates_res, int interleaved, const void* prev_c,
                                          float* cprev_res, float* cell_res, void* h_out, void* c_out,
                                          int n, int h, int w, int hid, int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_convlstm_gates_refresh";
  long long total = 0;
  int rc = check_dense(who, n, h, w, hid, dtype, &total);
  if (rc != MIE_OK) return rc;
  MIE_REQUIRE(gates_res && cprev_res && cell_res && h_out && c_out, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(!interleaved || hid % 8 == 0, MIE_ERR_INVALID_ARG,
              "%s: the gate-interleaved column order needs hid %% 8 == 0 (hid=%d)", who, hid);
  MIE_REQUIRE(cprev_res != cell_res && h_out != c_out, MIE_ERR_INVALID_ARG,
              "%s: cprev_res / cell_res and h_out / c_out must be distinct", who);
  MIE_REQUIRE(mie_aligned(gates_res, 4) && mie_aligned(prev_c, 4) && mie_aligned(cprev_res, 4) &&
                  mie_aligned(cell_res, 4) && mie_aligned(h_out, 4) && mie_aligned(c_out, 4),
              MIE_ERR_INVALID_ARG, "%s: buffers must be 4-byte aligned", who);
  const dim3 grid((unsigned)((total + 255) / 256));
  if (dtype == MIE_DTYPE_BF16)
    hipLaunchKernelGGL(k_convlstm_gates_refresh<mie_bf16>, grid, dim3(256), 0, (hipStream_t)stream, gates_res,
                       interleaved, (const mie_bf16*)prev_c, cprev_res, cell_res, (mie_bf16*)h_out,
                       (mie_bf16*)c_out, total, hid);
  else
    hipLaunchKernelGGL(k_convlstm_gates_refresh<float>, grid, dim3(256), 0, (hipStream_t)stream, gates_res,
                       interleaved, (const float*)prev_c, cprev_res, cell_res, (float*)h_out, (float*)c_out,
                       total, hid);
  return mie_check_launch(who);
}

extern "C" int mie_convgru_gates_refresh(const void* update, const void* cand, const void* prev_state,
                                         float* diff_res, float* update_res, void* new_state, int n, int h,
                                         int w, int hid, int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_convgru_gates_refresh";
  long long total = 0;
  int rc = check_dense(who, n, h, w, hid, dtype, &total);
  if (rc != MIE_OK) return rc;
  MIE_REQUIRE(update && cand && new_state, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(diff_res == nullptr || diff_res != update_res, MIE_ERR_INVALID_ARG,
              "%s: the two reservoirs must be distinct", who);
  MIE_REQUIRE(mie_aligned(update, 4) && mie_aligned(cand, 4) && mie_aligned(prev_state, 4) &&
                  mie_aligned(diff_res, 4) && mie_aligned(update_res, 4) && mie_aligned(new_state, 4),
              MIE_ERR_INVALID_ARG, "%s: buffers must be 4-byte aligned", who);
  const dim3 grid((unsigned)((total + 255) / 256));
  if (dtype == MIE_DTYPE_BF16)
    hipLaunchKernelGGL(k_convgru_gates_refresh<mie_bf16>, grid, dim3(256), 0, (hipStream_t)stream,
                       (const mie_bf16*)update, (const mie_bf16*)cand, (const mie_bf16*)prev_state, diff_res,
                       update_res, (mie_bf16*)new_state, total);
  else
    hipLaunchKernelGGL(k_convgru_gates_refresh<float>, grid, dim3(256), 0, (hipStream_t)stream,
                       (const float*)update, (const float*)cand, (const float*)prev_state, diff_res, update_res,
                       (float*)new_state, total);
  return mie_check_launch(who);
}

extern "C" int mie_mul_dense(const void* a, const void* b, void* out, long long count, int dtype, void* stream) {
  mie_clear_error();
  const char* who = "mie_mul_dense";
  long long total = 0;
  int rc = check_dense(who, 1, 1, 1, count, dtype, &total);
  if (rc != MIE_OK) return rc;
  MIE_REQUIRE(a && b && out, MIE_ERR_INVALID_ARG, "%s: NULL pointer", who);
  MIE_REQUIRE(mie_aligned(a, 4) && mie_aligned(b, 4) && mie_aligned(out, 4), MIE_ERR_INVALID_ARG,
              "%s: buffers must be 4-byte aligned", who);
  const dim3 grid((unsigned)((total + 255) / 256));
  if (dtype == MIE_DTYPE_BF16)
    hipLaunchKernelGGL(k_mul_dense<mie_bf16>, grid, dim3(256), 0, (hipStream_t)stream, (const mie_bf16*)a,
                       (const mie_bf16*)b, (mie_bf16*)out, total);
  else
    hipLaunchKernelGGL(k_mul_dense<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)a,
                       (const float*)b, (float*)out, total);
  return mie_check_launch(who);
}
