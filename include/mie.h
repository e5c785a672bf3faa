/*
 * mie.h -- C ABI of libmie_hip.so: masked incremental inference kernels for
 * AMD MI355X (gfx950).
 *
 * Every entry point takes raw device pointers, plain integers and a HIP
 * stream (passed as void* so that this header needs no HIP include), returns
 * an int status (MIE_OK == 0, negative on error) and never allocates device
 * memory, never synchronises with the host and never aborts.  After a
 * negative status mie_last_error_string() describes the failure (thread
 * local).  All launches are asynchronous on the given stream and contain no
 * host-side read of device data (launch bounds come from capacities, kernels
 * exit early on the device-side counts), so a sequence of calls can be
 * captured in a HIP graph.
 *
 * Layouts.  Delta tensors and reservoirs are fp32 NHWC ("channels_last"):
 * element (n, y, x, c) lives at ((n*H + y)*W + x)*C + c.  Pixel masks are
 * uint8 [N, H, W] (1 = the pixel carries a delta).  Filters use the layout
 * the reference extension takes, [Cin][K][K][Cout] (= weight.permute(1,2,3,0)
 * of a torch OIHW weight; reference: ext/pointops/pointops_functional.py:13-14).
 *
 * Tiles.  The image plane is cut into 8x8 pixel tiles (the output tile of
 * the reference 3x3 kernel, ext/pointops/_C_ext/pointops/ext_conv.cu:352);
 * tile id = (n*tiles_y + ty)*tiles_x + tx.  A tile set (mie_tileset) lists
 * the ids of the tiles that hold at least one active pixel, ascending.
 *
 * Clean-delta invariant.  Every delta buffer written by these kernels is
 * exactly zero outside the active pixels of its tile set, so it can be used
 * as a dense tensor by the caller.  To keep that invariant without touching
 * the whole frame, mie_build_mask_tiles also lists the tiles that were
 * active in the previous step and are not any more ("stale"); every kernel
 * that writes a delta over a tile set zeroes the stale tiles.
 */
#ifndef MIE_H_
#define MIE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MIE_OK 0
#define MIE_ERR_INVALID_ARG (-1)   /* null / misaligned pointer, bad size   */
#define MIE_ERR_UNSUPPORTED (-2)   /* kernel size / stride / shape not built */
#define MIE_ERR_CAPACITY (-3)      /* tile set too small for the geometry   */
#define MIE_ERR_LAUNCH (-4)        /* HIP reported a launch failure         */

#define MIE_TILE 8                 /* tile edge in pixels                   */

/* activation kinds of mie_act_incr / fused conv epilogue */
#define MIE_ACT_NONE 0
#define MIE_ACT_RELU 1
#define MIE_ACT_LEAKY_RELU 2
#define MIE_ACT_SIGMOID 3
#define MIE_ACT_TANH 4

/* footprint kinds of mie_build_mask_tiles */
#define MIE_FOOT_CONV 0    /* out(oy,ox) |= in(oy*s-p+ky, ox*s-p+kx)              */
#define MIE_FOOT_UP2X 1    /* bilinear x2, align_corners=False, non-zero weights  */
#define MIE_FOOT_TCONV 2   /* transposed conv: oy = iy*s - p + ky                 */

/* conv code path selection */
#define MIE_PATH_AUTO 0
#define MIE_PATH_VALU 1
#define MIE_PATH_MFMA 2

/* flags of mie_act_incr / mie_mul_incr */
#define MIE_FLAG_KEEP_RESERVOIR 1  /* compute the delta, leave reservoirs as is */

/* element type of the DELTA buffers of a call (inputs, outputs, addend, and the
 * matrix-core filter copy).  Reservoirs, bias, the plain filter and every
 * accumulation are fp32 in both cases.  bf16 values are converted with
 * round-to-nearest-even.  Pointers to such buffers are `void*` below. */
#define MIE_DTYPE_F32 0
#define MIE_DTYPE_BF16 1
/* fp32 deltas whose matrix-core contraction runs on the bf16 instruction at fp32 accuracy: every input and
 * weight is split into three bf16 terms (hi + mid + lo, all 24 significant bits) and the six term products
 * that matter are accumulated in fp32 -- what is dropped is at most 2^-23 of |x*w| per product and 2^-26
 * typically (an fp32 multiply-add rounds at 2^-24); measured against fp64, whole convs come out at 0.6 to 1.1
 * times the error of the fp32 matrix-core instruction.  Taken by mie_pack_filter and by the `dtype` of
 * mie_conv_masked / _ws / _noalloc, mie_conv_refresh, mie_upconv_masked, mie_conv_gates_masked (shapes:
 * mie_conv_f32x3_takes) and mie_tconv2x_masked / mie_tconv2x_refresh (c1, c2 multiples of 64), with filter_mc
 * packed for it; every buffer is what it is for MIE_DTYPE_F32.  Values must be finite and below the bf16
 * maximum (3.39e38): an infinity, or a value that rounds to one in bf16, splits into inf - inf and gives
 * NaN where the fp32 instruction would give an infinity. */
#define MIE_DTYPE_F32_BF16X3 2

/* frame kinds of mie_events_to_frame */
#define MIE_EVENTS_VOXEL 0      /* num_bins channels, linear weights in time   */
#define MIE_EVENTS_HISTOGRAM 1  /* 2 channels: counts of p == -1, of p == +1   */

/* counts[] slots of a tile set */
#define MIE_CNT_ACTIVE 0
#define MIE_CNT_STALE 1
#define MIE_CNT_TICKET 2
#define MIE_CNT_WORDS 4

/*
 * A tile set at resolution (n, h, w).  All pointers are device memory owned
 * by the caller; capacity = mie_tile_capacity(n, h, w) entries.  Zero-fill
 * counts[] and flags[] once before the first use (and again whenever the
 * delta buffers written under this tile set are re-zeroed by the caller).
 */
typedef struct mie_tileset {
  int32_t n, h, w;
  uint8_t* pixmask;   /* [n*h*w]      1 = active pixel                        */
  int32_t* tiles;     /* [capacity]   active tile ids, ascending              */
  int32_t* stale;     /* [capacity]   tiles active last step, inactive now    */
  int32_t* counts;    /* [MIE_CNT_WORDS] active, stale, ticket, reserved      */
  uint32_t* flags;    /* [capacity]   16-byte aligned; bit 0 = tile active,
                         bit 1 = active after the previous build        */
} mie_tileset;

/* Library version (major*10000 + minor*100 + patch). */
int mie_version(void);

/* Text of the last error on the calling thread ("" if none). */
const char* mie_last_error_string(void);

/* Number of 8x8 tiles of an (n, h, w) plane = capacity of its tile set. */
int mie_tile_capacity(int n, int h, int w);

/*
 * pixmask[n,y,x] = any_c(|delta[n,y,x,c]| > threshold).
 * Replaces: the reference's only mask definitions, max-pool of abs(x) against
 * a threshold with field size 1 (incr_modules/utils.py:22-25,
 * utils/str_sparse_utils.py:10-11); the dilation by the field is the
 * MIE_FOOT_CONV footprint of mie_build_mask_tiles.
 */
int mie_mask_from_delta(const void* delta, int n, int h, int w, int c,
                        float threshold, uint8_t* pixmask, int dtype, void* stream);

/*
 * Build the output pixel mask and the ordered active-tile list of an op from
 * the pixel mask(s) of its input(s).
 *   in_mask / in_mask2: uint8 [n, h_in, w_in]; in_mask NULL = every input
 *   pixel active; in_mask2 optional second input at the same resolution
 *   (skip sum / concat), OR-ed with the first.
 *   foot, k, stride, pad: footprint (MIE_FOOT_*); for MIE_FOOT_UP2X k, stride
 *   and pad are ignored.  Output resolution is out->h, out->w.
 * Writes out->pixmask (every pixel), out->flags, out->tiles (ascending ids),
 * out->stale (tiles that were active after the previous build of `out`, as
 * out->flags remembers it, and are not any more; ascending) and
 * out->counts[ACTIVE, STALE].
 * Aliasing: out->pixmask may be in_mask / in_mask2 only for the identity
 * footprint (MIE_FOOT_CONV, k = 1, stride = 1, pad = 0); any other footprint
 * reads neighbouring bytes while they are written and is refused with
 * MIE_ERR_INVALID_ARG.
 * Sets of 33 to 512 tiles are built in one launch: the workgroup that finishes last (a ticket in
 * out->counts[MIE_CNT_TICKET], zero between calls) ranks the lists; larger sets take a second launch for that.
 * Replaces: the mask argument of conv{1,3,5,7}x*_increment_ext
 * (ext/pointops/_C_ext/pointops/ops.cpp:27-48), which the reference kernel
 * never reads (ext_conv.cu:74-76 synthesises a fake one).
 */
int mie_build_mask_tiles(const uint8_t* in_mask, const uint8_t* in_mask2,
                         int h_in, int w_in, int foot, int k, int stride,
                         int pad, const mie_tileset* out, void* stream);

/*
 * mie_mask_from_delta(delta -> thr_mask) followed by mie_build_mask_tiles(thr_mask, in_mask2, conv footprint k /
 * stride / pad -> out) as ONE launch (two above 128 tiles: the lists then have a launch of their own), for networks whose
 * masks depend on values: a conv with
 * a thresholded input mask otherwise pays three or four launches of 4-14 us each before it can start.  delta is
 * [out->n, h_in, w_in, c] of `dtype` (MIE_DTYPE_F32 / MIE_DTYPE_BF16), 16-byte aligned; thr_mask [out->n, h_in, w_in]
 * receives the thresholded input mask (a pixel is active when |delta| > threshold in any channel), which the conv
 * takes as its input pixel mask; in_mask2 (may be NULL) is OR-ed in before the footprint, as in
 * mie_build_mask_tiles.  Results are bit-equal to the two calls.  Limits: stride + pad <= k and
 * 7 * stride + k <= 24 (MIE_ERR_UNSUPPORTED otherwise: use the two calls); thr_mask, in_mask2 and out->pixmask are
 * three distinct buffers.  Uses out->counts[MIE_CNT_TICKET], which is zero between calls.
 * Replaces: the mask a thresholded module derives from its input, maxpool(abs(x)) >= thr with field 1
 * (incr_modules/utils.py:22-25), chained with the footprint of the conv that reads it.
 */
int mie_build_mask_tiles_thresholded(const void* delta, int c, int dtype, float threshold, uint8_t* thr_mask,
                                     const uint8_t* in_mask2, int h_in, int w_in, int k, int stride, int pad,
                                     const mie_tileset* out, void* stream);

/*
 * A sequence of mie_build_mask_tiles calls as one launch: the tile sets of a whole network, whose structural
 * masks are all footprints of footprints of the input pixel mask.  ops[i] holds the arguments of the i-th call;
 * the result -- every out[i].pixmask, flags, tiles, stale, counts -- is what the n_ops calls would leave when
 * issued in order on the stream.  An in_mask / in_mask2 that is the pixmask of an earlier op's `out` is taken
 * from that op (the chain never goes through memory); any other is read from memory once.  All ops share one
 * batch size out.n.  One workgroup per sample walks the chain on bitmaps in LDS; with one sample and at most 4096
 * tiles per set that is the only launch, otherwise a second kernel ranks all the lists.
 * Limits: conv footprints of stride 1 or 2, transposed-conv footprints of stride 2 (MIE_ERR_UNSUPPORTED
 * otherwise); ops plus masks read from memory <= MIE_PLAN_MAX_STEPS, and the masks alive at one time must fit the
 * LDS of a workgroup as bitmaps (MIE_ERR_CAPACITY: split the plan, or fall back to mie_build_mask_tiles).  ops is
 * host memory, read during the call only.
 * Replaces: nothing in the reference, which propagates no masks (every module returns None in the mask slot,
 * incr_modules/mask_incr_modules.py:41,103,178); the mask definitions are those of mie_build_mask_tiles
 * (incr_modules/utils.py:22-25, utils/str_sparse_utils.py:10-11).
 */
#define MIE_PLAN_MAX_STEPS 40
typedef struct mie_plan_op {
  const uint8_t* in_mask;    /* as in mie_build_mask_tiles (NULL = every input pixel active) */
  const uint8_t* in_mask2;
  int32_t h_in, w_in;
  int32_t foot, k, stride, pad;
  mie_tileset out;
} mie_plan_op;

int mie_build_mask_plan(const mie_plan_op* ops, int n_ops, void* stream);

/*
 * mie_build_mask_plan with a cap on the workgroups of its first kernel, for a plan that runs BESIDE other kernels --
 * the next step's tile sets built on a second stream while this step's convs run.  A plan workgroup is 1024 threads
 * and most of a CU's LDS; at the default (up to 256 workgroups, one round of the chip) it takes the CUs from the
 * convs it runs beside: at 8x480x640 the first stride-2 encoder went from 43 to 107 us.  With 64 the plan takes
 * longer, which nothing waits for, and the step of 8 frames 2.20 instead of 2.25 ms.  Same results as
 * mie_build_mask_plan; max_workgroups > 0 (values above the default cap mean the default).
 * Replaces: nothing in the reference (see mie_build_mask_plan).
 */
int mie_build_mask_plan_wgs(const mie_plan_op* ops, int n_ops, int max_workgroups, void* stream);

/*
 * Re-order a fp32 [cin][k][k][cout] filter into the layout the matrix-core
 * kernels stream, so that the k-steps a lane multiplies per tap come as one
 * 16-byte load:
 *   MIE_DTYPE_F32  (cin % 8 == 0):  P[ci/8][tap][(ci%8)/4][co][ci%4], fp32
 *   MIE_DTYPE_BF16 (cin % 16 == 0): P[ci/16][tap][(ci%16)/8][co][ci%8], bf16
 *   MIE_DTYPE_F32_BF16X3 (cin % 16 == 0): P[ci/16][tap][term][(ci%16)/8][co][ci%8], bf16,
 *        term 0 / 1 / 2 = the weight rounded to bf16, the rest of it rounded to bf16, what is left
 * `packed` holds cin*k*k*cout elements of that type (three times that many bf16 for
 * MIE_DTYPE_F32_BF16X3); do this once per weight update.
 * Replaces: convert_filter_out_channels_last
 * (ext/pointops/pointops_functional.py:13-14), which plays the same role for
 * the reference kernel.
 */
int mie_pack_filter(const float* filter, int cin, int k, int cout, void* packed,
                    int dtype, void* stream);

/*
 * 1 if the matrix-core conv takes this shape with dtype MIE_DTYPE_F32_BF16X3 (k = 3 or 5 at stride 1 with
 * c1, c2 multiples of 32, or k = 5 at stride 2 with multiples of 16; cout a multiple of 32), else 0: such a call must then be made with MIE_DTYPE_F32 and the
 * fp32 filter copy.  No counterpart in the reference (it has one arithmetic, cuDNN's or its own
 * kernel's fp32: ext/pointops/_C_ext/pointops/ext_conv.cu:74-76).
 */
int mie_conv_f32x3_takes(int k, int stride, int c1, int c2, int cout);

/*
 * Masked convolution of a delta: for every active tile of `out`
 *   acc = conv2d(x (++ x2), filter, bias = none, stride, pad)
 * and then, with reservoir == NULL:      out_delta  = acc
 *        with reservoir != NULL:          r0 = reservoir; r1 = r0 + acc;
 *                                         reservoir = r1;
 *                                         out_delta = act(r1) - act(r0)
 * (the fused form of nnConvIncr followed by nnReservedActivation).
 * Stale tiles of `out` are zeroed in out_delta.  Inactive input pixels are
 * never read.  out->pixmask must hold every output pixel whose window contains
 * an active input pixel (mie_build_mask_tiles / mie_build_mask_plan make exactly
 * that set; a superset is fine): at the other pixels of an active tile acc is
 * zero by construction, and the matrix-core kernels write out_delta = 0 there
 * without touching the reservoir.  addend (optional, [n, h_out, w_out, cout]) is
 * added to acc first:
 * a clean delta whose active pixels lie in out->pixmask -- the residual of a
 * residual block, or the contribution of a few extra input channels computed
 * by another launch (conv over a concat = sum of convs over its parts).
 *   x  : [n, h_in, w_in, c1] delta with pixel mask xmask (NULL = all active),
 *        feeds filter input channels [0, c1)
 *   x2 : optional second input [n, h_in, w_in, c2] (NULL, c2 = 0 if absent),
 *        feeds filter input channels [c1, c1 + c2) -- the concat-free form of
 *        torch.cat((x, h), 1) in ConvLSTMIncr (incr_modules/e2depth_incr.py:100)
 *   filter : fp32 [cin_total][k][k][cout], c1 + c2 <= cin_total
 *   filter_mc : optional copy of the same filter in the matrix-core layout made
 *        by mie_pack_filter with the same dtype.  The MFMA kernels read only this copy;
 *        without it MIE_PATH_AUTO takes the VALU kernels and MIE_PATH_MFMA is
 *        refused.
 *   Aliasing: for k > 1 neither x nor x2 may be out_delta, and neither input
 *   mask may be out->pixmask (workgroups read the halo of their tile while
 *   others write it): MIE_ERR_INVALID_ARG.  The same holds for h_delta /
 *   c_delta of mie_conv_gates_masked.
 *   k in {1,3,5,7}, stride in {1,2}; out->h/w must equal (h_in+2*pad-k)/stride+1
 *   dtype : element type of x, x2, addend, out_delta and filter_mc
 *        (MIE_DTYPE_BF16: products of bf16 values accumulated in fp32 on the
 *        matrix cores, v_mfma_f32_32x32x16_bf16; the VALU kernels multiply the
 *        fp32 `filter`, so give them bf16-representable weights for one result)
 * Replaces: conv{1,3,5,7}x*_increment_ext(x_incr, mask, filter, out_incr, stride)
 * (ext/pointops/_C_ext/pointops/ops.cpp:51-114, include/ops.h:8-52) and the
 * F.conv2d fallback the reference actually runs
 * (incr_modules/mask_incr_modules.py:175-178).
 */
int mie_conv_masked(const void* x, const uint8_t* xmask, int c1,
                    const void* x2, const uint8_t* x2mask, int c2,
                    int h_in, int w_in, const float* filter,
                    const void* filter_mc, int cin_total,
                    int k, int stride, int pad, int cout,
                    const mie_tileset* out, void* out_delta,
                    const void* addend, float* reservoir, int act_kind,
                    float slope, int path, int dtype, void* stream);

/*
 * mie_conv_masked with a workspace.  On planes of very few tiles (a 16x16
 * plane is 4 tiles) a conv launch has too few workgroups for the chip; given a
 * workspace, the matrix-core path then splits the contraction of each
 * (tile, 32-channel slab) over up to 8 workgroups, which write fp32 partial
 * sums to the workspace, and a second kernel adds them in a fixed order and
 * runs the epilogue (results are reproducible run to run, and differ from the
 * unsplit launch by fp32 rounding of the regrouped sum only).
 *   workspace : device memory, 16-byte aligned, or NULL (then exactly
 *        mie_conv_masked); workspace_bytes its size.  A launch is split when
 *        k = 3 or 5, tiles x cout/32 <= 128 (tiles = mie_tile_capacity of `out`), the
 *        inputs are at least 4 staging chunks deep and the workspace holds at
 *        least 2 planes of n*h*w*cout floats (8 MiB covers 8 planes of every
 *        shape that qualifies); otherwise the workspace is not touched.
 *        Its contents are scratch: undefined after the call, and calls that
 *        share one workspace must be ordered (same stream).
 * Has no counterpart in the reference, whose convs run as one launch of
 * whatever size (ext/pointops/_C_ext/pointops/ext_conv.cu:74-76).
 */
int mie_conv_masked_ws(const void* x, const uint8_t* xmask, int c1,
                       const void* x2, const uint8_t* x2mask, int c2,
                       int h_in, int w_in, const float* filter,
                       const void* filter_mc, int cin_total,
                       int k, int stride, int pad, int cout,
                       const mie_tileset* out, void* out_delta,
                       const void* addend, float* reservoir, int act_kind,
                       float slope, int path, int dtype, void* workspace,
                       long long workspace_bytes, void* stream);

/*
 * mie_conv_masked_ws for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the
 * same arguments as mie_conv_masked, and the workspace of the split form is an
 * array of MIE_NOALLOC_WS_BYTES that lives in the library's device image (each
 * GPU the library runs on holds its own copy until the process ends).  The call
 * allocates and frees nothing; it looks the array's device address up once per
 * device, on the first call made with that device current (make that first
 * call outside of a stream capture).  Results are those of mie_conv_masked_ws
 * with a workspace of MIE_NOALLOC_WS_BYTES, bit for bit.
 *   Limit: two partial planes must fit, 2 * n*h*w*cout*4 <= MIE_NOALLOC_WS_BYTES
 *   (every launch the split form takes is far below that); a larger output is
 *   refused with MIE_ERR_CAPACITY and nothing is launched -- use
 *   mie_conv_masked there.
 *   Sharing: every call on a GPU uses that GPU's one array and leaves its last
 *   partial sums there.  Nothing in it has to start at zero (each launch
 *   writes every partial sum it later reads), but calls that overlap on one
 *   GPU (two streams, two threads) race on it: order them on one stream.
 * Has no counterpart in the reference; it exists for callers that cannot
 * allocate.
 */
#define MIE_NOALLOC_WS_BYTES (8 * 1024 * 1024)
int mie_conv_masked_noalloc(const void* x, const uint8_t* xmask, int c1,
                            const void* x2, const uint8_t* x2mask, int c2,
                            int h_in, int w_in, const float* filter,
                            const void* filter_mc, int cin_total,
                            int k, int stride, int pad, int cout,
                            const mie_tileset* out, void* out_delta,
                            const void* addend, float* reservoir, int act_kind,
                            float slope, int path, int dtype, void* stream);

/*
 * Dense refresh through the same kernels: for every active tile of `out`
 * (build it with in_mask = NULL so that every tile is active)
 *   y = conv2d(x (++ x2), filter, bias, stride, pad) (+ addend);
 *   reservoir = y (if reservoir != NULL);  out_dense = act(y)
 * bias may be NULL.  This is the dense pass that (re)fills the cached
 * pre-activations every 20-100 frames, and the dense comparator of the
 * incremental path.
 * Replaces: nnConvIncr.forward_refresh_reservoirs followed by
 * nnReservedActivation.forward_refresh_reservoirs
 * (incr_modules/mask_incr_modules.py:182-196,253-256).
 */
int mie_conv_refresh(const void* x, int c1, const void* x2, int c2, int h_in,
                     int w_in, const float* filter, const void* filter_mc,
                     int cin_total, int k,
                     int stride, int pad, int cout, const float* bias,
                     const mie_tileset* out, void* out_dense,
                     const void* addend, float* reservoir, int act_kind,
                     float slope, int path, int dtype, void* stream);

/*
 * Incremental point-wise non-linearity over the active tiles of ts:
 *   r0 = reservoir; r1 = r0 + in_delta; out_delta = act(r1) - act(r0);
 *   reservoir = r1   (in place)
 * in_delta is read at the active pixels of ts->pixmask only.  If
 * out_pixmask != NULL it receives the refined mask
 *   out_pixmask = ts->pixmask & any_c(out_delta != 0)   (all n*h*w bytes of
 * active and stale tiles are written; other tiles are left untouched, so
 * zero-fill it once), else the input mask is passed through by the caller.
 * flags & MIE_FLAG_KEEP_RESERVOIR: the reservoir is read only (the form of
 * NonlinearPointOpIncr.forward without the accumulate).
 * Replaces: activation_increment(X, in_incr, out_incr)
 * (ext/pointops/_C_ext/pointops/ops.cpp:8-23, pointop_cuda.cu:17-52) and
 * NonlinearPointOpIncr._nonlin + IncrementReserve.accumulate
 * (incr_modules/mask_incr_modules.py:101-103,248-251).
 */
int mie_act_incr(int act_kind, float slope, const void* in_delta,
                 float* reservoir, void* out_delta, int c,
                 const mie_tileset* ts, uint8_t* out_pixmask, int flags,
                 int dtype, void* stream);

/*
 * Delta quantiser ("k-fence"): lets multiples of k through and carries the rest
 * to later steps.  At the active pixels of ts->pixmask, per element
 *   t = carry + in_delta;  out_delta = k * floor(0.5 + t / k);  carry = t - out_delta
 * (each operation rounded on its own, true division: bit-identical to the same
 * expression in fp32 on the host); inactive pixels of active tiles and stale
 * tiles get out_delta = 0 and keep their carry.  k = *k_dev when k_dev != NULL
 * (a device scalar, so that a refresh can change k without a host read or a new
 * graph capture), else k_host; a k that is not positive and finite lets the
 * delta through unchanged.  A carry that started at zero stays within
 * [-k/2, k/2], where the dense expression emits 0 as well.  out_pixmask as in
 * mie_act_incr (refined mask any_c(out_delta != 0)): it is what makes the
 * following layers sparse again.  out_delta may alias in_delta.
 * Replaces: KFencedMaskModule.forward / floor_by_k
 * (incr_modules/mask_incr_modules.py:32-42); k is what
 * KFencedMaskModule.forward_refresh_reservoirs (:44-48) sets.
 */
int mie_kfence_incr(const void* in_delta, float* carry, const float* k_dev,
                    float k_host, void* out_delta, int c, const mie_tileset* ts,
                    uint8_t* out_pixmask, int dtype, void* stream);

/*
 * Incremental point-wise product (product rule with cached operands):
 *   out = (d2 + r2) * d1 + r1 * d2;  r1 += d1;  r2 += d2
 * d1/d2 are read only where their pixel masks m1/m2 (NULL = all active) are
 * set, ts must be built from the union of the two masks.
 * flags & MIE_FLAG_KEEP_RESERVOIR: r1, r2 are read only (the bare
 * IncrPointwiseMultiply of the reference).
 * Replaces: IncrPointwiseMultiply + nnReservedMultiplication.forward
 * (incr_modules/mask_incr_functional.py:52-54, mask_incr_modules.py:67-75).
 */
int mie_mul_incr(const void* d1, const uint8_t* m1, float* r1,
                 const void* d2, const uint8_t* m2, float* r2,
                 void* out_delta, int c, const mie_tileset* ts, int flags,
                 int dtype, void* stream);

/*
 * out = a + b over the active tiles of ts (built from the union of ma, mb).
 * Replaces: the skip sum / residual sum on deltas
 * (incr_modules/e2depth_incr.py:220,333).
 */
int mie_add_incr(const void* a, const uint8_t* ma, const void* b,
                 const uint8_t* mb, void* out_delta, int c,
                 const mie_tileset* ts, int dtype, void* stream);

/*
 * Incremental max pooling: over the active tiles of `out` (built with
 * MIE_FOOT_CONV for the same k / stride / pad)
 *   out_delta = maxpool(reservoir + in_delta) - maxpool(reservoir)
 * with torch's max_pool2d window rule (taps outside the image do not count).
 * The reservoir ([n,h_in,w_in,c] fp32) is only READ: pooling windows of
 * neighbouring tiles overlap, so the caller accumulates it afterwards with
 * mie_accumulate.  in_delta is read at the active pixels of in_mask only.
 * Replaces: nnMaxPool2dIncr.forward (incr_modules/mask_incr_modules.py:217-219).
 */
int mie_maxpool_incr(const void* in_delta, const uint8_t* in_mask,
                     const float* reservoir, int h_in, int w_in, int c, int k,
                     int stride, int pad, const mie_tileset* out, void* out_delta,
                     int dtype, void* stream);

/*
 * reservoir += in_delta at the active pixels of ts (nothing else is touched).
 * Replaces: IncrementReserve.accumulate
 * (incr_modules/mask_incr_functional.py:40-44), a dense add_ over the frame.
 */
int mie_accumulate(const void* in_delta, float* reservoir, int c,
                   const mie_tileset* ts, int dtype, void* stream);

/*
 * Bilinear x2 up-sampling (align_corners = False) of a delta, optionally of
 * the sum of two deltas: out = up2x(a + b).  `out` is the tile set at the
 * output resolution (2*h_in, 2*w_in), built with MIE_FOOT_UP2X.
 * Replaces: interpolate_from_module (incr_modules/mask_incr_functional.py:76-78)
 * with the skip sum of UNetRecurrentIncr.forward folded in
 * (incr_modules/e2depth_incr.py:429-431).
 */
int mie_upsample2x_incr(const void* a, const uint8_t* ma, const void* b,
                        const uint8_t* mb, int h_in, int w_in, int c,
                        const mie_tileset* out, void* out_delta, int dtype,
                        void* stream);

/*
 * Two independent mie_upsample2x_incr calls of the same geometry (c channels,
 * [n,h_in,w_in] -> twice that) in one launch: input, mask, tile set and output
 * of their own each.  For decoders that up-sample the parts of a channel
 * concat one by one (incr_modules/evflownet_incr.py:294-343 up-samples the
 * concatenated tensor; here the concat is never formed).
 */
int mie_upsample2x_pair_incr(const void* a0, const uint8_t* m0,
                             const mie_tileset* out0, void* out_delta0,
                             const void* a1, const uint8_t* m1,
                             const mie_tileset* out1, void* out_delta1,
                             int h_in, int w_in, int c, int dtype, void* stream);

/*
 * Fused incremental ConvLSTM gate math for hidden size hid over the active
 * tiles of ts.  gates_delta is [n,h,w,4*hid] in the reference chunk order
 * [in, remember, out, cell] (incr_modules/e2depth_incr.py:103).  State kept
 * by the caller (all [n,h,w,*] fp32, updated in place):
 *   gates_res [4*hid]  pre-activation gate reservoirs
 *   cprev_res [hid]    cached previous cell state (operand of m2)
 *   cell_res  [hid]    cached new cell state (input of tanh2)
 * cprev_delta (with mask cprev_mask) may be NULL = zero.  Computes, per
 * element, exactly the chain sigmoid1..3/tanh1 -> m1 + m2 -> tanh2 -> m3 of
 * ConvLSTMIncr.forward with post-activation operands recomputed from the
 * pre-activation reservoirs, and writes h_delta, c_delta ([n,h,w,hid]).
 * Replaces: incr_modules/e2depth_incr.py:103-120 (about 25 ATen launches).
 */
int mie_convlstm_gates_incr(const void* gates_delta, float* gates_res,
                            const void* cprev_delta, const uint8_t* cprev_mask,
                            float* cprev_res, float* cell_res, void* h_delta,
                            void* c_delta, int hid, const mie_tileset* ts,
                            int dtype, void* stream);

/*
 * Fused incremental ConvGRU gate math for hidden size hid over the active
 * tiles of ts, for a cell whose state is reset every step (the only way the
 * reference runs it: new_state = candidate * update, incr_modules/
 * evflownet_incr.py:58-69 with prev_state None).  gates_delta is
 * [n,h,w,2*hid]: the delta of the update-gate conv in channels [0, hid) and of
 * the candidate (out-gate) conv in [hid, 2*hid) -- ONE mie_conv_masked with
 * the two filters stacked along the output channels, both convs read the same
 * input.  State kept by the caller ([n,h,w,hid] fp32, updated in place):
 *   update_res  pre-activation reservoir of the update gate (sigmoid)
 *   cand_res    pre-activation reservoir of the candidate (tanh)
 * Computes, per element, sigmoid / tanh increments on those reservoirs and the
 * product rule of nnReservedMultiplication with its cached operands recomputed
 * from them, and writes h_delta ([n,h,w,hid]).
 * Replaces: the second gate conv, two activation increments and the
 * incremental multiply of ConvGRUIncr.forward
 * (incr_modules/evflownet_incr.py:58-69, mask_incr_modules.py:67-75).
 */
int mie_convgru_gates_incr(const void* gates_delta, float* update_res,
                           float* cand_res, void* h_delta, int hid,
                           const mie_tileset* ts, int dtype, void* stream);

/*
 * The gates conv of a ConvLSTM and its gate chain in ONE kernel: the 3x3,
 * stride 1, pad 1 conv of mie_conv_masked (x ++ x2 -> 4*hid channels) whose
 * epilogue is mie_convlstm_gates_incr, so that the 4*hid-channel gate delta is
 * never written to memory.  Matrix-core path only: needs filter_mc, c1 and c2
 * in whole staging chunks (32 channels fp32, 64 bf16) and hid % 8 == 0;
 * otherwise MIE_ERR_UNSUPPORTED (use the two calls then).
 *   filter / filter_mc / gates_res : the 4*hid output columns are NOT in the
 *     order [in | remember | out | cell] x hid of the two-call form but
 *     interleaved by gate: column 4*hc + g  <->  gate g of hidden channel hc,
 *     so that one workgroup owns all four gates of its hidden channels and
 *     reads / writes them as one 16-byte access.  gates_res
 *     ([n,h,w,4*hid]) lives in that order too (a refresh through
 *     mie_conv_refresh with the same filter and a bias in the same order fills
 *     it consistently).
 *   cprev_* / cell_res / h_delta / c_delta ([n,h,w,hid]) as in
 *     mie_convlstm_gates_incr, plain channel order.
 * Replaces: incr_modules/e2depth_incr.py:100-120 (cat, conv, chunk, the chain).
 */
int mie_conv_gates_masked(const void* x, const uint8_t* xmask, int c1,
                          const void* x2, const uint8_t* x2mask, int c2,
                          int h_in, int w_in, const float* filter,
                          const void* filter_mc, int cin_total, int hid,
                          const mie_tileset* out, float* gates_res,
                          const void* cprev_delta, const uint8_t* cprev_mask,
                          float* cprev_res, float* cell_res, void* h_delta,
                          void* c_delta, int dtype, void* stream);

/*
 * mie_conv_gates_masked with a workspace.  On planes of few tiles (tiles x 4*hid/32 <= 128, inputs at least 4 staging
 * chunks deep) the contraction runs as a split 3x3 conv of the two inputs -- up to 8 workgroups per (tile, 32-column
 * slab) write fp32 partial sums of the gate columns to the workspace -- and a second kernel adds them in a fixed order
 * and runs the gate chain.  workspace NULL (workspace_bytes 0): exactly mie_conv_gates_masked.  Workspace rules as
 * in mie_conv_masked_ws.  No counterpart in the reference (incr_modules/e2depth_incr.py:100-120 is one conv launch).
 */
int mie_conv_gates_masked_ws(const void* x, const uint8_t* xmask, int c1,
                             const void* x2, const uint8_t* x2mask, int c2,
                             int h_in, int w_in, const float* filter,
                             const void* filter_mc, int cin_total, int hid,
                             const mie_tileset* out, float* gates_res,
                             const void* cprev_delta, const uint8_t* cprev_mask,
                             float* cprev_res, float* cell_res, void* h_delta,
                             void* c_delta, int dtype, void* workspace,
                             long long workspace_bytes, void* stream);

/*
 * Dense refresh of a ConvLSTM cell after its gates conv: gates_res
 * ([n,h,w,4*hid] fp32) holds the gate pre-activations mie_conv_refresh wrote --
 * in the order [in | remember | out | cell] x hid, or (interleaved != 0) in the
 * gate-interleaved order of mie_conv_gates_masked.  Per (pixel, hidden channel):
 *   cell = sigmoid(in) * tanh(cell_gate) + sigmoid(remember) * prev_c
 *   h_out = sigmoid(out) * tanh(cell);  c_out = cell
 *   cprev_res = prev_c;  cell_res = cell      (the reservoirs of the gate chain)
 * prev_c ([n,h,w,hid], element type `dtype`) may be NULL = zero state, and may
 * be c_out (the previous refresh's cell state, updated in place); h_out / c_out
 * are dense tensors of that type.
 * Replaces: the state math of ConvLSTMIncr.forward_refresh_reservoirs
 * (incr_modules/e2depth_incr.py:144-166) and its reservoir clones
 * (incr_modules/mask_incr_functional.py:46-48).
 */
int mie_convlstm_gates_refresh(const float* gates_res, int interleaved,
                               const void* prev_c, float* cprev_res,
                               float* cell_res, void* h_out, void* c_out, int n,
                               int h, int w, int hid, int dtype, void* stream);

/*
 * Dense refresh of a ConvGRU cell after its gate convs: update = sigmoid(update
 * gate), cand = tanh(out gate), both dense [n,h,w,hid] of type `dtype` as the
 * fused conv refresh returns them; prev_state may be NULL = zero.
 *   new_state = prev_state + (cand - prev_state) * update
 *   diff_res = cand - prev_state;  update_res = update   (optional: the cached
 *   operands of the incremental product, nnReservedMultiplication)
 * new_state may be prev_state (updated in place).
 * Replaces: incr_modules/evflownet_incr.py:84-96.
 */
int mie_convgru_gates_refresh(const void* update, const void* cand,
                              const void* prev_state, float* diff_res,
                              float* update_res, void* new_state, int n, int h,
                              int w, int hid, int dtype, void* stream);

/*
 * out[i] = a[i] * b[i] for count dense elements of type `dtype` (out may alias a
 * or b): prev_state * reset in front of the candidate conv of a ConvGRU refresh
 * (incr_modules/evflownet_incr.py:90).
 */
int mie_mul_dense(const void* a, const void* b, void* out, long long count,
                  int dtype, void* stream);

/*
 * Per-channel scale of a delta over the active tiles of ts: out = in * scale[c]
 * (inactive pixels of active tiles and stale tiles get zeros).  scale is fp32 [c];
 * for an eval-mode batch norm it is weight / sqrt(running_var + eps).
 * out_delta may alias in_delta.
 * Replaces: bn2d_from_module (incr_modules/mask_incr_functional.py:69-73), the
 * body of nnBatchNorm2dIncr.forward (incr_modules/mask_incr_modules.py:200-207).
 */
int mie_scale_incr(const void* in_delta, const float* scale, void* out_delta,
                   int c, const mie_tileset* ts, int dtype, void* stream);

/*
 * Adaptive average pooling of a delta [n,h_in,w_in,c] to [n,h_out,w_out,c] with
 * torch's window rule (output index o covers [floor(o*in/out), ceil((o+1)*in/out))).
 * Pixels whose in_mask byte is 0 are not read and add nothing (in_mask NULL =
 * all active); the divisor is the window size.  Every output element is written.
 * Replaces: nnAdaptiveAvgPool2dIncr.forward
 * (incr_modules/mask_incr_modules.py:228-233).
 */
int mie_avgpool_incr(const void* in_delta, const uint8_t* in_mask, int n, int h_in,
                     int w_in, int c, int h_out, int w_out, void* out_delta,
                     int dtype, void* stream);

/*
 * Fully connected layer on a delta, bias dropped: out[n][o] = sum_i in[n][i] *
 * W[o][i].  weight_t is the TRANSPOSED weight, fp32 [f_in][f_out] (make it once
 * per weight update), so that an input feature's contribution is one contiguous
 * row; rows of features whose delta is exactly 0 are not read.
 * Replaces: nnLinearIncr.forward (incr_modules/mask_incr_modules.py:106-116).
 */
int mie_linear_incr(const void* in_delta, int n, int f_in, const float* weight_t,
                    int f_out, void* out_delta, int dtype, void* stream);

/*
 * Bilinear x2 up-sampling (align_corners = False) of a + b followed by the 5x5
 * stride-1 pad-2 conv of mie_conv_masked, in one kernel: the up-sampled tensor
 * is never written.  a (mask amask) and the optional b (mask bmask) are
 * [n,h_in,w_in,c] deltas at HALF the output resolution; `out` is the conv's tile
 * set at (2*h_in, 2*w_in), built from the up-sampled mask (MIE_FOOT_UP2X, then
 * MIE_FOOT_CONV).  Matrix-core path only, two forms:
 *   - filter_mc given, c a multiple of the staging chunk (32 fp32 / 64 bf16
 *     channels), cout of 32, k = 5, pad = 2;
 *   - a single input (b = NULL) of c <= 8 channels, k = 3 or 5, pad = k/2, cout
 *     a multiple of 32 (filter_mc unused): the 2-channel flow estimate in front
 *     of an EVFlowNet-incr decoder (incr_modules/evflownet_incr.py:463-470);
 * otherwise MIE_ERR_UNSUPPORTED (use mie_upsample2x_incr + mie_conv_masked).
 * Epilogue (addend, reservoir, activation) as in mie_conv_masked.
 * Replaces: interpolate_from_module + nnConvIncr.forward of
 * UpsampleConvLayerIncr.forward with the skip sum in front of it
 * (incr_modules/e2depth_incr.py:306-313, 429-431).
 */
int mie_upconv_masked(const void* a, const uint8_t* amask, const void* b,
                      const uint8_t* bmask, int c, int h_in, int w_in,
                      const float* filter, const void* filter_mc, int cin_total,
                      int k, int pad, int cout, const mie_tileset* out,
                      void* out_delta, const void* addend, float* reservoir,
                      int act_kind, float slope, int dtype, void* stream);

/*
 * mie_upconv_masked with a workspace, as mie_conv_masked_ws is to mie_conv_masked: on planes of few tiles (tiles x
 * cout/32 <= 128, c at least 4 staging chunks) the contraction of each (tile, 32-channel slab) is split over up to 8
 * workgroups that write fp32 partial sums to the workspace, and a second kernel adds them in a fixed order and runs the
 * epilogue.  workspace NULL (workspace_bytes 0): exactly mie_upconv_masked.  The few-channel form is never split.
 * No counterpart in the reference (one launch per conv whatever its size, incr_modules/e2depth_incr.py:306-313).
 */
int mie_upconv_masked_ws(const void* a, const uint8_t* amask, const void* b,
                         const uint8_t* bmask, int c, int h_in, int w_in,
                         const float* filter, const void* filter_mc, int cin_total,
                         int k, int pad, int cout, const mie_tileset* out,
                         void* out_delta, const void* addend, float* reservoir,
                         int act_kind, float slope, int dtype, void* workspace,
                         long long workspace_bytes, void* stream);

/*
 * The tail of E2Depth-incr in one kernel: the last decoder -- mie_upconv_masked, 5x5 over up2x(a + b), c = 64 -> cout =
 * 32 channels, reservoir + activation -- whose activation increment y is NOT stored, followed by the one-channel 1x1
 * prediction conv over y + skip (skip: the head's output delta, [n, 2*h_in, 2*w_in, cout], clean outside skip_mask, NULL
 * mask = every pixel), the update of the prediction's pre-activation reservoir and its activation increment:
 *   r1 = reservoir + conv;  y = act(r1) - act(reservoir)  (rounded to the delta type);  reservoir = r1
 *   z  = sum_c pred_filter[c] * y[c] + pred_filter[cout + c] * skip[c]
 *   p1 = pred_reservoir + z;  pred_delta = pred_act(p1) - pred_act(pred_reservoir);  pred_reservoir = p1
 * at every pixel of the active tiles of `out`, zeros in pred_delta ([n, 2*h_in, 2*w_in], element type `dtype`) on its
 * stale tiles.  `out` is the tile set of the PREDICTION: the union of the decoder's output set and the set of skip
 * (mie_build_mask_tiles with both as inputs, MIE_FOOT_CONV k = 1); the decoder's conv runs on all of its tiles.
 * pred_filter: fp32 [2][cout], the prediction conv's weights for y and for skip (the same row twice for
 * pred(x + head)).  Implemented for MIE_DTYPE_BF16, c = 64, cout = 32, decoder activations none / ReLU / leaky ReLU,
 * on planes of 2048 .. 2^20 tiles; MIE_ERR_UNSUPPORTED otherwise (run mie_upconv_masked and mie_conv_masked).
 * Replaces: the last UpsampleConvLayerIncr, the skip sum, the prediction layer and the output activation of
 * UNetRecurrentIncr.forward (incr_modules/e2depth_incr.py:429-435).
 */
int mie_upconv_pred_masked(const void* a, const uint8_t* amask, const void* b,
                           const uint8_t* bmask, int c, int h_in, int w_in,
                           const float* filter, const void* filter_mc, int cin_total,
                           int cout, const mie_tileset* out, float* reservoir,
                           int act_kind, float slope, const void* skip,
                           const uint8_t* skip_mask, const float* pred_filter,
                           float* pred_reservoir, int pred_act, float pred_slope,
                           void* pred_delta, int dtype, void* stream);

/*
 * Masked transposed convolution of a delta (stride s, padding p; the output
 * size out->h/w fixes output_padding): out(oy,ox,co) = sum x(iy,ix,ci) *
 * filter[ci][ky][kx][co] over oy = iy*s - p + ky, ox = ix*s - p + kx, with
 * the same reservoir/activation epilogue as mie_conv_masked.  filter is the
 * torch ConvTranspose2d weight [Cin][Cout][K][K] permuted to [Cin][K][K][Cout].
 * `out` must be built with MIE_FOOT_TCONV.
 * Replaces: transposed_conv2d_from_module
 * (incr_modules/mask_incr_functional.py:64-66).
 */
int mie_tconv_masked(const void* x, const uint8_t* xmask, int cin, int h_in,
                     int w_in, const float* filter, int k, int stride, int pad,
                     int cout, const mie_tileset* out, void* out_delta,
                     float* reservoir, int act_kind, float slope, int dtype,
                     void* stream);

/*
 * The decoder case of mie_tconv_masked on the matrix cores: stride 2, kernel size k
 * in {3, 5}, padding k/2, output exactly twice the input (output_padding 1), over
 * one or two inputs (x ++ x2, the concat-free form of a decoder that takes
 * torch.cat of its parts, incr_modules/evflownet_incr.py:463-470).  The four
 * sub-pixel phases of the output are four stride-1 contractions over disjoint
 * tap subsets of the same staged input, so no product is spent on inserted zeros.
 *   x / x2 : [n,h_in,w_in,c1] / [n,h_in,w_in,c2] deltas with their pixel masks
 *        (x2 optional); c1, c2 multiples of 32 (bf16 and MIE_DTYPE_F32_BF16X3: 64), cout of 32
 *   filter / filter_mc : [cin_total][k][k][cout] as in mie_tconv_masked and its
 *        matrix-core copy (mie_pack_filter, required); c1 + c2 <= cin_total
 *   out    : output tile set at (2*h_in, 2*w_in), built with MIE_FOOT_TCONV
 *        (k, stride 2, pad k/2) from the OR of the input masks
 *   blocks : tile set at (h_in, w_in) of the 16x16 output blocks the workgroups
 *        walk, built from out->pixmask with MIE_FOOT_CONV k = 2, stride 2, pad 0
 *   addend, reservoir, act_kind, slope : epilogue of mie_conv_masked (addend:
 *        e.g. the contribution of a few more input channels computed by
 *        mie_tconv_masked, covered by `out`)
 *   workspace / workspace_bytes : as in mie_conv_masked_ws (planes of very few
 *        blocks split their contraction over up to 8 workgroups); may be NULL
 * Replaces: transposed_conv2d_from_module
 * (incr_modules/mask_incr_functional.py:64-66) inside TransposedConvLayerIncr
 * (incr_modules/e2depth_incr.py:243-282).
 */
int mie_tconv2x_masked(const void* x, const uint8_t* xmask, int c1,
                       const void* x2, const uint8_t* x2mask, int c2, int h_in,
                       int w_in, const float* filter, const void* filter_mc,
                       int cin_total, int k, int cout, const mie_tileset* out,
                       const mie_tileset* blocks, void* out_delta,
                       const void* addend, float* reservoir, int act_kind,
                       float slope, int dtype, void* workspace,
                       long long workspace_bytes, void* stream);

/*
 * Dense refresh twin of mie_tconv2x_masked: out_dense = act(tconv(x ++ x2) +
 * bias (+ addend)) with `out` and `blocks` all active (build both with in_mask =
 * NULL), reservoir (optional) = the pre-activation.
 * Replaces: the conv_transpose2d + bias of TransposedConvLayerIncr's refresh
 * (incr_modules/e2depth_incr.py:275-282).
 */
int mie_tconv2x_refresh(const void* x, int c1, const void* x2, int c2, int h_in,
                        int w_in, const float* filter, const void* filter_mc,
                        int cin_total, int k, int cout, const float* bias,
                        const mie_tileset* out, const mie_tileset* blocks,
                        void* out_dense, const void* addend, float* reservoir,
                        int act_kind, float slope, int dtype, void* stream);

/*
 * Dense refresh twin of mie_tconv_masked, as mie_conv_refresh is of
 * mie_conv_masked: out_dense = act(tconv(x) + bias) over the active tiles of
 * `out` (build it with in_mask = NULL: every tile), reservoir (optional) = the
 * pre-activation.
 * Replaces: the conv_transpose2d + bias of TransposedConvLayerIncr's refresh
 * (incr_modules/e2depth_incr.py:275-282).
 */
int mie_tconv_refresh(const void* x, int cin, int h_in, int w_in,
                      const float* filter, int k, int stride, int pad, int cout,
                      const float* bias, const mie_tileset* out, void* out_dense,
                      float* reservoir, int act_kind, float slope, int dtype,
                      void* stream);

/*
 * Event front end: scatter raw events into a frame, or directly into the DELTA
 * between the frames of two time windows, in the layout the network consumes.
 *   events : [n_events][4] doubles (t, x, y, p), the reference's .npy row
 *            layout; t * t_scale is in the unit of start_* / delta_t
 *            (t_scale = 1e-9 for nanosecond stamps, util.py:90).  Events off the
 *            sensor are skipped.
 *   window : an event belongs to a window iff start < t*t_scale < start + delta_t.
 *   MIE_EVENTS_VOXEL: ts = (num_bins-1)*(t*t_scale-start)/delta_t; p*(1-frac(ts))
 *            goes to bin floor(ts), p*frac(ts) to the next bin, p == 0 counts as
 *            -1 (events_to_voxel_grid_absT, data_fetchers/utils/util.py:78-107;
 *            with start = first stamp, delta_t = last - first, t_scale = 1 it is
 *            events_to_voxel_grid, :110-152).
 *   MIE_EVENTS_HISTOGRAM: channel 0 counts p == -1, channel 1 counts p == +1
 *            (event_histogram, util.py:62-75).
 *   delta  : 0 -> out = frame of the window at start_new (start_old unused);
 *            1 -> out = frame(start_new) - frame(start_old), each event of
 *            either window visited once (replaces forming both frames and
 *            `event_tensor - event_tensor_prev`,
 *            run_e2depth_continuous_dataset.py:66).
 *   pad_*  : ReflectionPad2d((left, right, top, bottom)) applied to the result
 *            (run_e2depth_continuous_dataset.py:49), folded into the scatter.
 *   out    : fp32 [height+pad_top+pad_bottom][width+pad_left+pad_right][channels]
 *            (one NHWC sample; offset the pointers per sample of a batch),
 *            fully rewritten (zero where no event lands).
 *   pixmask: same pixels, 1 where at least one contributing event landed.
 * Sums use floating-point atomics: a pixel hit by several events can differ in
 * the last bits between runs (the histogram kind is exact).
 */
int mie_events_to_frame(const double* events, int n_events, int kind, int num_bins,
                        int height, int width, int pad_left, int pad_right,
                        int pad_top, int pad_bottom, double t_scale,
                        double start_old, double start_new, double delta_t,
                        int delta, float* out, uint8_t* pixmask, void* stream);

/*
 * mie_events_to_frame with the frame also delivered as bf16, for the networks that run on bf16 deltas
 * (MIE_DTYPE_BF16): `sums` is the fp32 frame exactly as mie_events_to_frame leaves it in `out` (the
 * atomic sums need fp32), `out` [same shape] receives every element of it rounded to nearest even, in
 * the same stream -- the cast a caller would otherwise run as a separate pass over the frame
 * (`event_tensor.to(...)` after data_fetchers/utils/util.py:107).  out != sums, 8-byte aligned.
 */
int mie_events_to_frame_bf16(const double* events, int n_events, int kind, int num_bins,
                             int height, int width, int pad_left, int pad_right,
                             int pad_top, int pad_bottom, double t_scale,
                             double start_old, double start_new, double delta_t,
                             int delta, float* sums, void* out, uint8_t* pixmask, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MIE_H_ */
