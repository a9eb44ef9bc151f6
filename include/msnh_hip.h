/*
 * msnh_hip.h -- C ABI of the MI355X (gfx950) kernel library `libmsnh_hip.so`.
 *
 * This is the drop-in boundary of the convolutional hot path: everything Msnhnet's layers do on the
 * device (its CUDA kernels, cuBLAS and cuDNN calls) is reached through the plain-C entry points below.
 * No C++ or framework types cross it: pointers are raw device (or, where stated, host) addresses, sizes
 * are ints, streams/events/graphs are opaque `void*` handles owned by this library.
 *
 * Conventions
 *   - Every function returns 0 on success and a non-zero code on failure; it never exits the process
 *     (the reference prints and calls exit(), src/config/MsnhnetCuda.cpp:18-56).  The text of the last
 *     failure on the calling thread is returned by msnh_hip_last_error().
 *   - Activations live on the device in NHWC ("channels-last") order: element (n,y,x,c) of a tensor is at
 *     data[((n*H + y)*W + x)*ld + c], ld >= C being the pixel stride in elements.  ld > C lets a tensor be
 *     a channel slice of a wider buffer, which is how route/concat layers are planned away.  The reference
 *     keeps NCHW (src/layers/MsnhConvolutionalLayer.cpp:645-760); NCHW float32 remains the layout of
 *     everything that enters or leaves the library (msnh_hip_nchw_to_nhwc / msnh_hip_nhwc_to_nchw).
 *   - dtype is MSNH_F32 or MSNH_F16 (IEEE half).  Arithmetic is always accumulated in float32.
 *   - Shapes are validated on the host before any launch; a shape the kernels cannot run is an error,
 *     never an out-of-bounds access.
 */
#ifndef MSNH_HIP_H
#define MSNH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *msnh_stream_t;   /* hipStream_t; NULL = the library's default stream */
typedef void *msnh_event_t;    /* hipEvent_t */
typedef void *msnh_graph_t;    /* instantiated hipGraphExec_t */

enum msnh_dtype { MSNH_F32 = 0, MSNH_F16 = 1 };

/* Same numeric values as the reference's ActivationType (include/Msnhnet/config/MsnhnetCfg.h:95-120). */
enum msnh_act
{
    MSNH_ACT_LOGISTIC = 0,
    MSNH_ACT_RELU     = 1,
    MSNH_ACT_RELU6    = 2,
    MSNH_ACT_LEAKY    = 8,
    MSNH_ACT_SWISH    = 16,
    MSNH_ACT_HARD_SWISH = 17,
    MSNH_ACT_MISH     = 18,
    MSNH_ACT_NONE     = 22
};

enum msnh_conv_algo
{
    MSNH_CONV_AUTO      = 0,   /* let the library choose */
    MSNH_CONV_DIRECT    = 1,   /* one thread per output element; any shape; the fallback */
    MSNH_CONV_IGEMM     = 2,   /* implicit GEMM on MFMA, LDS-staged tiles; needs (in_c/groups) % 8 == 0 (f16) or % 4 (f32) */
    MSNH_CONV_DEPTHWISE = 3,   /* groups == in_c == out_c, bandwidth-bound direct kernel */
    MSNH_CONV_WINOGRAD  = 4,   /* F(2x2,3x3): ksize 3, stride 1, dilation 1, groups 1 */
    MSNH_CONV_STEM      = 5,   /* in_c <= 4 first layer: reads NCHW float32 input directly (cast fused) */
    MSNH_CONV_POINTWISE = 7,   /* 1x1 stride 1, float16, in_c and out_c <= 128 and multiples of 8: weights resident in LDS, pixels
                                  straight from memory into MFMA fragments, no tiles (tile must be 0).  IGEMM weight packing.
                                  Never chosen by AUTO. */
    MSNH_CONV_IGEMM_SPLITK = 6,/* IGEMM with the K loop cut into up to 8 slices on separate workgroups, float32 partial sums in
                                  the workspace summed in slice order (deterministic); for launches with few output tiles.
                                  Same weight packing as IGEMM.  Never chosen by AUTO. */
    MSNH_CONV_STEM_DOWN = 8,   /* not an algorithm of msnh_hip_conv2d: the label of a launch of msnh_hip_conv_stem_down (first layer
                                  and first stride-2 layer as one), so that plans and timing tables can name it */
    MSNH_CONV_WINOGRAD_FUSED = 9, /* F(2x2,3x3) in one launch, float16 in and out, in_c a multiple of 16: input transform into LDS, the 16
                                  products with all accumulators in registers, output transform in the epilogue; weights packed as
                                  for MSNH_CONV_WINOGRAD, no workspace */
    MSNH_CONV_IGEMM_TAIL = 11, /* not an algorithm of msnh_hip_conv2d: the label of a launch of msnh_hip_conv2d_tail (a convolution and the 1x1
                                  convolution that reads its result) */
    MSNH_CONV_MBCONV = 10      /* not an algorithm of msnh_hip_conv2d: the label of a launch of msnh_hip_mbconv (1x1 expand, 3x3 depthwise
                                  and 1x1 project convolution of an inverted-residual block as one) */
};

/* ------------------------------------------------------------------------------------------------
 * Runtime plumbing.  Replaces the reference's `Cuda` helper class (src/config/MsnhnetCuda.cpp:105-239:
 * cudaSetDevice, getCudaStream, mallocCudaArray/makeCudaArray, pushCudaArray/pullCudaArray, freeCuda).
 * ---------------------------------------------------------------------------------------------- */
const char *msnh_hip_last_error(void);
int msnh_hip_init(int device);                                  /* selects the device, creates the default stream */
int msnh_hip_device_count(int *count);
int msnh_hip_device_name(char *dst, int cap, int *cu_count, size_t *total_mem);
int msnh_hip_malloc(void **dptr, size_t bytes);
int msnh_hip_free(void *dptr);
int msnh_hip_host_alloc(void **hptr, size_t bytes);             /* pinned host memory */
int msnh_hip_host_free(void *hptr);
int msnh_hip_memcpy_h2d(void *dst, const void *src, size_t bytes, msnh_stream_t s);
int msnh_hip_memcpy_d2h(void *dst, const void *src, size_t bytes, msnh_stream_t s);
int msnh_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, msnh_stream_t s);
int msnh_hip_fill_zero(void *dst, size_t bytes, msnh_stream_t s); /* a fill kernel, safe under graph capture */
int msnh_hip_stream_create(msnh_stream_t *s);
int msnh_hip_stream_destroy(msnh_stream_t s);
int msnh_hip_stream_sync(msnh_stream_t s);
int msnh_hip_event_create(msnh_event_t *e);
int msnh_hip_event_destroy(msnh_event_t e);
int msnh_hip_event_record(msnh_event_t e, msnh_stream_t s);
int msnh_hip_stream_wait_event(msnh_stream_t s, msnh_event_t e);   /* work queued on s afterwards starts once e has fired */
int msnh_hip_event_sync(msnh_event_t e);
int msnh_hip_event_elapsed_ms(msnh_event_t start, msnh_event_t stop, float *ms);
/* Stream capture into a replayable graph: every kernel launched on `s` between begin and end is
 * recorded instead of run.  No counterpart in the reference (it launches kernel by kernel,
 * src/net/MsnhNetBuilder.cpp:847). */
int msnh_hip_graph_begin(msnh_stream_t s);
int msnh_hip_graph_end(msnh_stream_t s, msnh_graph_t *g);
int msnh_hip_graph_launch(msnh_graph_t g, msnh_stream_t s);
int msnh_hip_graph_destroy(msnh_graph_t g);

/* ------------------------------------------------------------------------------------------------
 * Convolution.  Replaces ConvolutionalLayer::forwardGPU (src/layers/MsnhConvolutionalLayer.cpp:914-1183):
 * cudnnConvolutionForward (:995-1015) or im2ColExKernel + cublasSgemm (src/core/cuda/MsnhGemmGPU.cu:6-55,
 * 136-145), then convBnKernel (src/layers/cuda/MsnhConvolutionalLayerGPU.cu:6-24) or addBiasKernel
 * (src/core/cuda/MsnhBlasGPU.cu:656-688), then activateArrayKernel (src/layers/cuda/MsnhActivationsGPU.cu),
 * and -- when has_residual -- the axpy + activation of the enclosing Res/Res2/Add block
 * (src/layers/MsnhResBlockLayer.cpp:261-262, 264-293), all in one launch:
 *
 *     v = act( acc * scale[oc] + shift[oc] )                     acc = cross-correlation, float32
 *     if has_residual:  v = act2( v + res_mul * residual )
 *     y = out_mul * v
 *
 * Batch-norm is supplied folded: scale = gamma/sqrt(var+eps), shift = beta - gamma*mean/sqrt(var+eps)
 * (src/layers/MsnhConvolutionalLayer.cpp:811-815); plain bias is scale = 1 (or scale == NULL), shift = bias.
 * res_mul / out_mul are exact power-of-two rescalings used to keep float16 activations in range.
 * Output size must satisfy out = (in + 2*pad - (dilation*(ksize-1)+1))/stride + 1 (:388-398).
 * ---------------------------------------------------------------------------------------------- */
typedef struct msnh_conv_desc
{
    int   dtype;        /* of x, w and residual */
    int   out_dtype;    /* of y */
    int   batch, in_h, in_w, in_c, in_ld;
    int   out_c, out_h, out_w, out_ld;
    int   ksize, stride, pad, dilation, groups;
    int   act;          /* msnh_act of the conv layer itself */
    float act_param;    /* leaky slope */
    int   has_residual;
    int   res_ld;
    int   act2;         /* msnh_act applied after the residual add */
    float act2_param;
    float res_mul;
    float out_mul;
    int   algo;         /* msnh_conv_algo */
    int   tile;         /* IGEMM only: 0 = library default, 1..msnh_hip_conv2d_tile_count() = forced tile configuration */
    int   out_upsample; /* 0 or 1: y is [batch][out_h][out_w].  2 (MSNH_CONV_IGEMM only, no residual, out_c and out_ld multiples of 8): every
                           result pixel is written to the 2 x 2 pixels it maps to under nearest-neighbour upsampling, y is
                           [batch][2 out_h][2 out_w] -- the convolution in front of an UpSampleLayer (src/layers/MsnhUpSampleLayer.cpp:96-118,
                           Blas::cpuUpSample with stride 2 and scale 1) writes the upsampled tensor itself */
    int   xcd_blocks;   /* IGEMM algorithms, ungrouped and unsplit: how the tiles of the launch are dealt to the 8 XCDs (each has an L2 of its
                           own).  1: an XCD takes a run of pixel tiles with all their channel tiles (every input pixel is fetched into
                           one L2, every filter into all eight).  2, 4, 8: the XCDs form a g x (8 / g) grid over (channel tiles, pixel
                           tiles) and each fetches only its share of the filters and of the input.  0: the library takes the arrangement
                           that fetches the fewest bytes (MSNH_NO_XCD_BLOCKS=1 in the environment: always 1).  Same result bits either
                           way; no counterpart in the reference */
} msnh_conv_desc;

/* Number of tile configurations of the IGEMM algorithm; any of them computes the same result, they differ in
 * speed per shape.  The host library times them per layer at load (the reference asks cuDNN for the fastest
 * algorithm the same way, src/layers/MsnhConvolutionalLayer.cpp:150-194). */
int msnh_hip_conv2d_tile_count(void);
/* Version of the layouts msnh_hip_conv2d_pack_weights writes: packed weights kept on disk are valid for the version they were made under. */
int msnh_hip_conv2d_pack_layout_version(void);
/* 1 if IGEMM tile configuration `tile` can run this shape (some configurations are specialised, e.g. for 3x3
 * stride-1 layers whose input patch fits in LDS), else 0.  Pure host function. */
int msnh_hip_conv2d_tile_supported(const msnh_conv_desc *d, int tile);
/* Which algorithm MSNH_CONV_AUTO resolves to for this shape (never AUTO).  Pure host function. */
int msnh_hip_conv2d_select_algo(const msnh_conv_desc *d);
/* Number of elements (of d->dtype) of the packed weight buffer for `algo`.  Pure host function. */
size_t msnh_hip_conv2d_packed_weight_elems(const msnh_conv_desc *d, int algo);
/* Host-side weight packing from the `.msnhbin` order w[out_c][in_c/groups][k][k] float32
 * (src/layers/MsnhConvolutionalLayer.cpp:1255-1257) into the layout `algo` reads:
 *   DIRECT / IGEMM : [out_c][k*k][in_c/groups], tap-major, channel fastest
 *   DEPTHWISE      : [k*k][channels]
 *   WINOGRAD       : [16][out_c][in_c]  = G g G^T per (oc,ic), G of F(2x2,3x3)
 *   STEM           : [k*k*in_c][out_c] float32 regardless of dtype
 * `packed` is host memory of msnh_hip_conv2d_packed_weight_elems() elements; upload it afterwards. */
int msnh_hip_conv2d_pack_weights(const msnh_conv_desc *d, int algo, const float *oihw, void *packed);
/* Scratch bytes `workspace` must provide for `algo` (0 for all but WINOGRAD). */
size_t msnh_hip_conv2d_workspace_bytes(const msnh_conv_desc *d, int algo);
/* x: NHWC d->dtype (STEM: NCHW float32); w: packed for the resolved algo; scale/shift: float32[out_c] or NULL;
 * residual: NHWC d->dtype with pixel stride res_ld, or NULL; y: NHWC d->out_dtype with pixel stride out_ld. */
int msnh_hip_conv2d(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift,
                    const void *residual, void *y, void *workspace, size_t workspace_bytes, msnh_stream_t s);

/* A convolution and the 1x1 stride-1 pad-0 convolution that reads its result, as one launch, float16: the 3x3 convolution that closes a
 * Darknet residual block together with the 1x1 convolution that opens the next block (two ConvolutionalLayer::forwardGPU calls,
 * src/layers/MsnhConvolutionalLayer.cpp:984-1169, inside ResBlockLayer::forwardGPU, src/layers/MsnhResBlockLayer.cpp:215-302, with the
 * block's output read back from device memory between them).  d describes the first convolution as for msnh_hip_conv2d (algo MSNH_CONV_IGEMM,
 * ungrouped, out_c <= 256 and a multiple of 8; d->tile: 0 or one of the tiles that carry a tail, the last msnh_hip_conv2d_tile_count() -
 * msnh_hip_conv2d_tail_tile_first() + 1 ones); y is written as by msnh_hip_conv2d unless t->write_y is 0 (nobody else reads it).  Then
 * z = out_mul * act(scale2 * (w2 . y) + shift2) with y as rounded to float16, so that z carries the bits a separate launch reading y
 * would compute in the same k order.  w2: the 1x1 filters packed as for MSNH_CONV_IGEMM, [t->out_c][d->out_c] float16; t->out_c <= 128
 * and a multiple of 8; z: NHWC float16 with pixel stride t->out_ld (a multiple of 8), 16-byte aligned.  _supported: pure host function. */
typedef struct msnh_conv_tail_desc
{
    int   out_c, out_ld;
    int   act;          /* msnh_act of the 1x1 convolution */
    float act_param;
    float out_mul;
    int   write_y;
} msnh_conv_tail_desc;
int msnh_hip_conv2d_tail_tile_first(void);
int msnh_hip_conv2d_tail_supported(const msnh_conv_desc *d, const msnh_conv_tail_desc *t, int tile);
int msnh_hip_conv2d_tail(const msnh_conv_desc *d, const msnh_conv_tail_desc *t, const void *x, const void *w, const float *scale, const float *shift,
                         const void *residual, void *y, const void *w2, const float *scale2, const float *shift2, void *z, msnh_stream_t s);

/* The first two convolutions of the Darknet-53 / CSPDarknet-53 trunks as one launch, float16: a 3x3 stride-1 pad-1 convolution with 32
 * filters over the 3-channel NCHW float32 network input, then a 3x3 stride-2 pad-1 convolution with c2 = 32 / 64 / 128 filters
 * (two ConvolutionalLayer::forwardGPU calls, src/layers/MsnhConvolutionalLayer.cpp:984-1169, with the full-resolution 32-channel tensor
 * in device memory between them; here it stays in LDS).  y = out_mul * act2(scale2 * conv2(mid) + shift2) with
 * mid = float16(mid_mul * act1(scale1 * conv1(x) + shift1)); scale2 must undo mid_mul.  y: NHWC float16 [batch][(h+1)/2][(w+1)/2] with pixel
 * stride y_ld.  w1: [32][3][3][3], w2: [c2][32][3][3] float32 in `.msnhbin` order, packed by msnh_hip_conv_stem_down_pack into
 * msnh_hip_conv_stem_down_packed_elems(c2, 0 | 1) float16 elements each (upload them afterwards).  _supported: pure host function. */
int msnh_hip_conv_stem_down_supported(int in_c, int c1, int k1, int s1, int p1, int c2, int k2, int s2, int p2);
size_t msnh_hip_conv_stem_down_packed_elems(int c2, int which);
int msnh_hip_conv_stem_down_pack(const float *w1, int c2, const float *w2, void *packed1, void *packed2);
int msnh_hip_conv_stem_down(int batch, int h, int w, const float *x, const void *packed1, const float *scale1, const float *shift1, int act1,
                            float act1_param, float mid_mul, int c2, const void *packed2, const float *scale2, const float *shift2, int act2,
                            float act2_param, float out_mul, void *y, int y_ld, msnh_stream_t s);
/* The same launch followed, inside it, by the 1x1 stride-1 convolution with c3 = 32 filters that reads its result -- the opening of Darknet-53's
 * first residual block (a third ConvolutionalLayer::forwardGPU call, src/layers/MsnhConvolutionalLayer.cpp:984-1169, inside
 * ResBlockLayer::forwardGPU, src/layers/MsnhResBlockLayer.cpp:215-302): z = z_mul * act3(scale3 * (w3 . y) + shift3) over y as rounded to
 * float16 and stored (y is written as by msnh_hip_conv_stem_down: the block's residual add reads it), k in channel order as a separate launch
 * sums it.  w3: [32][c2] float32 in `.msnhbin` order, packed by msnh_hip_conv_stem_down_tail_pack into msnh_hip_conv_stem_down_tail_packed_elems(c2)
 * float16 elements; z: NHWC float16 with pixel stride z_ld (a multiple of 8), 16-byte aligned.  _supported: pure host function. */
int msnh_hip_conv_stem_down_tail_supported(int c2, int c3, int k3, int s3, int p3);
size_t msnh_hip_conv_stem_down_tail_packed_elems(int c2);
int msnh_hip_conv_stem_down_tail_pack(int c2, const float *w3, void *packed3);
int msnh_hip_conv_stem_down_tail(int batch, int h, int w, const float *x, const void *packed1, const float *scale1, const float *shift1, int act1,
                                 float act1_param, float mid_mul, int c2, const void *packed2, const float *scale2, const float *shift2, int act2,
                                 float act2_param, float out_mul, void *y, int y_ld, const void *packed3, const float *scale3, const float *shift3,
                                 int act3, float act3_param, float z_mul, void *z, int z_ld, msnh_stream_t s);

/* The inverted-residual block of MobileNetV2 as one launch, float16 NHWC: 1x1 convolution in_c -> exp_c, 3x3 depthwise convolution
 * (stride 1 or 2, pad 1) over the exp_c channels, 1x1 convolution exp_c -> out_c, each with its folded batch-norm and activation, then the
 * block's residual add (three ConvolutionalLayer::forwardGPU calls, src/layers/MsnhConvolutionalLayer.cpp:984-1169, the second with
 * groups == channels, inside a Res2BlockLayer / AddBlockLayer, src/layers/MsnhRes2BlockLayer.cpp forwardGPU; in the reference the
 * widened tensors live in device memory between the calls, here they stay in LDS):
 *   e = float16(mul1 * act1(scale1 * conv1x1(x) + shift1));   d = float16(mul2 * act2(scale2 * dw3x3(e) + shift2));
 *   y = out_mul * act4(act3(scale3 * conv1x1(d) + shift3) + res_mul * residual)      (without a residual: out_mul * act3(...))
 * scale2 must undo mul1 and scale3 must undo mul2 (the power-of-two scales of the two widened tensors).
 * Limits: in_c, out_c <= 96, all channel counts and pixel strides multiples of 8; _supported is a pure host function. */
typedef struct msnh_mbconv_desc {
    int batch, in_h, in_w, in_c, in_ld;
    int exp_c, stride;
    int out_c, out_h, out_w, out_ld;
    int act1, act2, act3, act4;
    float act1_param, act2_param, act3_param, act4_param;
    int has_residual, res_ld;
    float mul1, mul2, out_mul, res_mul;
} msnh_mbconv_desc;
int msnh_hip_mbconv_supported(const msnh_mbconv_desc *d);
/* Bytes of the packed weights (0: block not supported). */
size_t msnh_hip_mbconv_packed_bytes(const msnh_mbconv_desc *d);
/* w_expand: [exp_c][in_c], w_dw: [exp_c][3][3], w_project: [out_c][exp_c] float32 in `.msnhbin` order; scale1 / shift1 / scale2 / shift2:
 * float32[exp_c] or NULL (1 / 0).  `packed` is host memory of msnh_hip_mbconv_packed_bytes() bytes; upload it afterwards.  The packed record
 * depends on the channel counts, act1, act2, mul1 and mul2 of the descriptor (the scales of the widened tensors are folded into the first
 * two affines where the activation allows it): pack with the descriptor the launch will use. */
int msnh_hip_mbconv_pack(const msnh_mbconv_desc *d, const float *w_expand, const float *scale1, const float *shift1, const float *w_dw,
                         const float *scale2, const float *shift2, const float *w_project, void *packed);
/* x: NHWC float16 [batch][in_h][in_w] with pixel stride in_ld; scale3 / shift3: float32[out_c] on the device or NULL; residual: NHWC float16
 * with the output's geometry and pixel stride res_ld, or NULL; y: NHWC float16 with pixel stride out_ld. */
int msnh_hip_mbconv(const msnh_mbconv_desc *d, const void *x, const void *packed, const float *scale3, const float *shift3, const void *residual,
                    void *y, msnh_stream_t s);

/* ------------------------------------------------------------------------------------------------
 * Element-wise / bandwidth-bound layers (all NHWC, any ld).
 * ---------------------------------------------------------------------------------------------- */
/* y = out_mul * act( x*scale[c] + shift[c] ).  Stand-alone BatchNormLayer::forwardGPU
 * (src/layers/MsnhBatchNormLayer.cpp:284-398: copy + normKernel + scaleBias + addBias + activation). */
int msnh_hip_affine_act(int dtype, int out_dtype, long long pixels, int c, const void *x, int x_ld, const float *scale,
                        const float *shift, int act, float act_param, float out_mul, void *y, int y_ld, msnh_stream_t s);
/* y = out_mul * act( a_mul*a + b_mul*b ).  Res/Res2/AddBlock tail when it cannot be fused into a conv
 * (BlasGPU::gpuAxpy + gpuCopy + activation, src/layers/MsnhResBlockLayer.cpp:370-389). */
int msnh_hip_add_act(int dtype, long long pixels, int c, const void *a, int a_ld, float a_mul, const void *b, int b_ld,
                     float b_mul, int act, float act_param, float out_mul, void *y, int y_ld, msnh_stream_t s);
/* y[.., 0:c] = mul * x[.., 0:c].  Route / ConcatBlock copies that could not be planned away
 * (BlasGPU::gpuSimpleCopy, src/layers/MsnhRouteLayer.cpp:200-260). */
int msnh_hip_copy_channels(int dtype, long long pixels, int c, const void *x, int x_ld, float mul, void *y, int y_ld,
                           msnh_stream_t s);
/* Max pooling, padding = -FLT_MAX (maxpoolNormalKernel, src/layers/cuda/MsnhMaxPoolLayerGPU.cu:35-90 /
 * cudnnPoolingForward, src/layers/MsnhMaxPoolLayer.cpp:460-463). */
int msnh_hip_maxpool(int dtype, int batch, int in_h, int in_w, int c, const void *x, int x_ld, int ksize, int stride,
                     int pad, int out_h, int out_w, void *y, int y_ld, msnh_stream_t s);
/* `steps` (2 or 3) stride-1 max-pools of window ksize (3 or 5) and padding ksize / 2, the first over x, each further one over the
 * result of the one before it, in one launch; pool i writes y[i] (row stride y_ld[i]).  What the reference runs as separate layers
 * over one tensor in its SPP blocks -- windows 5, 9 and 13 (src/layers/MsnhMaxPoolLayer.cpp:293-345 called three times from
 * src/layers/MsnhConcatBlockLayer.cpp:255-355) are 5 over 5 over 5 -- with the same results as msnh_hip_maxpool called per pool.
 * msnh_hip_maxpool_chain_supported says whether the geometry is taken (the H x W tile of an image must fit LDS). */
int msnh_hip_maxpool_chain_supported(int dtype, int in_h, int in_w, int c, int ksize, int steps);
int msnh_hip_maxpool_chain(int dtype, int batch, int in_h, int in_w, int c, int ksize, int steps, const void *x, int x_ld, void *const *y,
                           const int *y_ld, msnh_stream_t s);
/* Average over the valid window elements (localAvgPoolNormalKernel, src/layers/cuda/MsnhLocalAvgPoolLayerGPU.cu:5;
 * CPU semantics src/layers/MsnhLocalAvgPoolLayer.cpp:286-344).  y = out_mul * mean. */
int msnh_hip_avgpool(int dtype, int out_dtype, int batch, int in_h, int in_w, int c, const void *x, int x_ld, int ksize,
                     int stride, int pad, int out_h, int out_w, float out_mul, void *y, int y_ld, msnh_stream_t s);
/* Nearest-neighbour upsample y[oy][ox] = scale * x[oy/stride][ox/stride] (upSampleKernel,
 * src/core/cuda/MsnhBlasGPU.cu:541-578, without its fill + accumulate). */
int msnh_hip_upsample_nearest(int dtype, int batch, int in_h, int in_w, int c, const void *x, int x_ld, int stride,
                              float scale, void *y, int y_ld, msnh_stream_t s);
/* Constant padding of the two image axes (PaddingLayer::forward, src/layers/MsnhPaddingLayer.cpp:143-177):
 * y[oy][ox] = mul * x[oy-top][ox-left] inside the image, `value` outside.  out_h/out_w = in + top + down / left + right. */
int msnh_hip_pad(int dtype, int batch, int in_h, int in_w, int c, const void *x, int x_ld, int top, int left, int out_h,
                 int out_w, float mul, float value, void *y, int y_ld, msnh_stream_t s);
/* Strided slice of channels, rows and columns (SliceLayer::forward, src/layers/MsnhSliceLayer.cpp:120-147):
 * y[oc][oy][ox] = mul * x[c0 + oc*cs][h0 + oy*hs][w0 + ox*ws]. */
int msnh_hip_slice(int dtype, int batch, int in_h, int in_w, const void *x, int x_ld, int c0, int cs, int h0, int hs, int w0,
                   int ws, int out_c, int out_h, int out_w, float mul, void *y, int y_ld, msnh_stream_t s);
/* Bilinear resize, source index (o + 0.5) * in/out - 0.5 clamped at 0 (align_corners 0) or o * (in-1)/(out-1)
 * (align_corners 1), float32 weights (Blas::cpuBilinearResize, src/core/MsnhBlas.cpp:2400-2465).  y = mul * value. */
int msnh_hip_upsample_bilinear(int dtype, int batch, int in_h, int in_w, int c, const void *x, int x_ld, int out_h, int out_w,
                               int align_corners, float mul, void *y, int y_ld, msnh_stream_t s);
/* Softmax over all pixels*c values of each image: e_i = exp(x_i/T - max/T), y_i = y_mul * e_i / sum e
 * (SoftMaxLayer::forward with groups 1, src/layers/MsnhSoftMaxLayer.cpp:60-93; Blas::softmax, src/core/MsnhBlas.cpp:1970-2110).
 * x_mul undoes the input's power-of-two storage scale. */
int msnh_hip_softmax(int dtype, int batch, int pixels, int c, const void *x, int x_ld, float x_mul, float temperature, void *y,
                     int y_ld, float y_mul, msnh_stream_t s);
/* Second half of a transposed convolution (the first half is a 1x1 msnh_hip_conv2d with ksize*ksize*c output channels,
 * channel = (ky*ksize + kx)*c + oc, weights W1[that channel][ic] = W[ic][oc][ky][kx]): output pixel (oy, ox) sums the taps whose
 * source pixel ((oy + pad - ky)/stride, (ox + pad - kx)/stride) exists, then y = out_mul * act(cols_mul * sum + bias)
 * (Gemm::cpuCol2Im, src/core/MsnhGemm.cpp:115-154; DeConvolutionalLayer::forward, src/layers/MsnhDeConvolutionalLayer.cpp:140-200).
 * out_h = (in_h - 1)*stride - 2*pad + ksize. */
int msnh_hip_deconv_col2im(int dtype, int batch, int in_h, int in_w, int c, int ksize, int stride, int pad, const void *cols, int cols_ld,
                           float cols_mul, const float *bias, int act, float act_param, int out_h, int out_w, float out_mul, void *y,
                           int y_ld, msnh_stream_t s);
/* Fully connected layer out[b][o] = act( sum_i x[b][i]*w[o][i] + bias[o] ) (cublasSgemm NT + bias,
 * src/layers/MsnhConnectedLayer.cpp:300-360).  x: [batch][inputs] d-type; w: [outputs][inputs] dtype;
 * y: float32 [batch][outputs].  x_mul undoes the input's power-of-two storage scale. */
int msnh_hip_connected(int dtype, int batch, int inputs, int outputs, const void *x, float x_mul, const void *w,
                       const float *bias, int act, float act_param, float *y, msnh_stream_t s);
/* Layout/dtype conversion at the library boundary (fp32ToFp16Kernel / fp16ToFp32Kernel,
 * src/config/cuda/MsnhnetCuda.cu:6-36, plus the transposition).  mul scales on the way. */
int msnh_hip_nchw_to_nhwc(int out_dtype, int batch, int c, int h, int w, const float *x_nchw, float mul, void *y,
                          int y_ld, msnh_stream_t s);
int msnh_hip_nhwc_to_nchw(int dtype, int batch, int c, int h, int w, const void *x, int x_ld, float mul, float *y_nchw,
                          msnh_stream_t s);

/* Letterbox of one 8-bit RGB image (HWC, device memory) into the network's NCHW float32 input: pad to a square with
 * 127, bilinear resize, optional R<->B swap, scale to [0,1] (half_init 0) or [-1,1].  Replaces
 * CVUtil::getPaddingZeroF32C3 (src/utils/MsnhCVUtil.cpp:203-261) + the host-to-device copy of the float image. */
int msnh_hip_letterbox_u8(const unsigned char *rgb_hwc, int width, int height, int net_w, int net_h, int half_init,
                          int shuffle_rgb, float *out_chw, msnh_stream_t s);
/* The reference's other 8-bit image -> network input variants (the PredDataType values of its C facade,
 * src/c_api/MsnhnetLib.h:11-20, each a CVUtil function): plain bilinear resize to (net_w, net_h) (MatOp::resize,
 * src/cv/MsnhCVMatOp.cpp:142-160, 404-437), optional R<->B swap, then per channel k
 *   MSNH_PRE_F32C3        u / 255                                       CVUtil::getImgDataF32C3, src/utils/MsnhCVUtil.cpp:91-138
 *   MSNH_PRE_F32C3_HALF   (u - 127.5) / 127.5                           the same with halfInit
 *   MSNH_PRE_GOOGLENET    u / 255 * (std_k / 0.5) + (mean_k - 0.5) / 0.5 with the ImageNet constants, getGoogLenetF32C3, :146-195
 *   MSNH_PRE_TRANSFORMED  (u / 255 - mean3[k]) / std3[k]                getTransformedF32C3, :269-318
 *   MSNH_PRE_CAFFE        u - {123.68, 116.779, 103.939}[k]             getCaffeModeF32C3, :326-375
 *   MSNH_PRE_PADDING_ZERO / _HALF   the letterbox above (msnh_hip_letterbox_u8 with half_init 0 / 1).
 * mean3 / std3 are host pointers, read at the call; only MSNH_PRE_TRANSFORMED needs them. */
enum msnh_preproc
{
    MSNH_PRE_F32C3 = 0, MSNH_PRE_F32C3_HALF = 1, MSNH_PRE_GOOGLENET = 2, MSNH_PRE_TRANSFORMED = 3, MSNH_PRE_CAFFE = 4,
    MSNH_PRE_PADDING_ZERO = 5, MSNH_PRE_PADDING_ZERO_HALF = 6
};
int msnh_hip_image_u8_to_input(const unsigned char *rgb_hwc, int width, int height, int net_w, int net_h, int kind,
                               const float *mean3, const float *std3, int shuffle_rgb, float *out_chw, msnh_stream_t s);

/* ------------------------------------------------------------------------------------------------
 * YOLO.  One launch per head replaces YoloLayer::forwardGPU's 15 launches (exSigmoidKernel, aExpTKernel,
 * sigmoidKernel: src/layers/cuda/MsnhYoloLayerGPU.cu:4-54, src/layers/MsnhYoloLayer.cpp:164-185) and
 * YoloOutLayer::forwardGPU's shuffleDataKernel + candidate threshold (src/layers/cuda/MsnhYoloOutLayerGPU.cu:5-21,
 * src/layers/MsnhYoloOutLayer.cpp:216-260).
 *   x        : head logits NHWC, channel = anchor*(5+classes)+m, times x_mul gives the true logit
 *   decoded  : float32, element (b,anchor,pixel,m) at decoded[b*decoded_batch_stride + ((anchor*h*w)+pixel)*(5+classes) + m]
 *              (the reference's "shuffled" order; the stride lets all heads of an image share one buffer)
 *   yolo_version : 3 or 4: centre (s + cell)*ratio, size anchor*e^t; 5: centre (2s - 0.5 + cell)*ratio, size anchor*(2s)^2
 *              (src/layers/MsnhYoloLayer.cpp:84-136)
 *   cand_idx : optional int32 [batch][cand_cap]; receives (anchor*h*w + pixel) + cand_base of every entry
 *              with objectness > conf_thresh, in no particular order;
 *   cand_cnt : int32 [batch], incremented by the number of entries found (caller zeroes it).
 * ---------------------------------------------------------------------------------------------- */
int msnh_hip_yolo_decode(int dtype, int batch, int h, int w, int classes, const void *x, int x_ld, float x_mul,
                         const float *anchors6, float ratio, int yolo_version, float *decoded, long long decoded_batch_stride,
                         float conf_thresh, int *cand_idx, int cand_cap, int cand_base, int *cand_cnt, msnh_stream_t s);
/* The same candidate list as msnh_hip_yolo_decode, but only the rows of the candidates are decoded (into the places the full
 * decode would give them; the rest of `decoded` is left as it is): an objectness scan over the head, then one row per
 * candidate.  For callers that only consume the candidates.  Arguments as for msnh_hip_yolo_decode; cand_idx and cand_cnt are
 * required.  rows, if not NULL: [batch][cand_cap][8] float32; the compact row of every candidate of this head is written at the
 * candidate's position in the list, exactly what msnh_hip_yolo_gather would produce for it (that call is then unnecessary).
 * decoded may be NULL when rows is given: nothing but the compact rows is written then. */
int msnh_hip_yolo_decode_candidates(int dtype, int batch, int h, int w, int classes, const void *x, int x_ld, float x_mul,
                                    const float *anchors6, float ratio, int yolo_version, float *decoded,
                                    long long decoded_batch_stride, float conf_thresh, int *cand_idx, int cand_cap, int cand_base,
                                    int *cand_cnt, float *rows, msnh_stream_t s);
/* msnh_hip_yolo_decode_candidates for all heads of a network in two launches instead of two per head (YoloLayer::forwardGPU of every head,
 * src/layers/MsnhYoloLayer.cpp:164-185, plus the candidate threshold of src/layers/MsnhYoloOutLayer.cpp:216-260): same list (as
 * a set: the order inside the list is arbitrary in both) and same rows.  heads[k].cand_base must be the sum of 3*h*w of the heads
 * before it (the cells of an image are numbered head after head); at most 4 heads; decoded may be NULL.  cand_cnt is
 * incremented by the number of candidates found (caller zeroes it). */
typedef struct msnh_yolo_head
{
    const void *x;          /* head logits NHWC, as for msnh_hip_yolo_decode */
    int x_ld;
    float x_mul;
    int h, w;
    float anchors[6];
    float ratio;
    int cand_base;
} msnh_yolo_head;
int msnh_hip_yolo_decode_candidates_heads(int dtype, int batch, int classes, int n_heads, const msnh_yolo_head *heads, int yolo_version,
                                          float *decoded, long long decoded_batch_stride, float conf_thresh, int *cand_idx, int cand_cap,
                                          int *cand_cnt, float *rows, msnh_stream_t s);
/* Candidate compaction for YoloOutLayer (the per-box part of src/layers/MsnhYoloOutLayer.cpp:120-170 done on
 * the device so that only surviving boxes cross PCIe): for image b and k < min(cand_cnt[b], cand_cap) reads
 * the decoded row of cell cand_idx[b][k] (rows are `5+classes` floats, row r of image b at
 * decoded + b*decoded_batch_stride + r*(5+classes)) and writes rows[b][k][0..7] =
 * { x, y, w, h, objectness, best class score, best class index, cell index } (the two indices as float;
 * best class = first maximum like std::max_element). */
int msnh_hip_yolo_gather(int batch, int classes, const float *decoded, long long decoded_batch_stride, const int *cand_idx,
                         int cand_cap, const int *cand_cnt, float *rows, msnh_stream_t s);
/* Per-class greedy NMS over the compact rows (src/layers/MsnhYoloOutLayer.cpp:175-194 and :381-461 on the device, so that
 * only the boxes that survive cross PCIe).  rows / cand_cap / cand_cnt as written by msnh_hip_yolo_gather or
 * msnh_hip_yolo_decode_candidates.  kept: [kept_cap][12] float32, 16-byte aligned; kept_cnt: int32 [1 + batch], zeroed by
 * the caller.  workspace: msnh_hip_yolo_nms_workspace_bytes() bytes of device memory (contents irrelevant), or NULL.
 * On return kept_cnt[0] is the number of records written (kept_cap >= batch * cand_cap can never overflow) and
 * kept_cnt[1 + b] != 0 says that image b was NOT processed completely: a class with more candidates in that image than the
 * kernels take (6144 with a workspace, 1024 without) or a NaN score.  The caller then runs the reference's procedure on
 * that image's rows itself and ignores its records.
 * A workspace of msnh_hip_yolo_nms_pair_workspace_bytes() bytes (16-byte aligned) gives the same results faster when a class has
 * thousands of members: the pair tests of such a class are then spread over the whole device as a bit matrix (a pool of at most
 * 64 MiB inside the workspace; a class whose matrix does not fit into what is left of it is handled by one workgroup as with the
 * plain workspace).
 * A record = { row[0..7], score of the class's best-scoring candidate, that candidate's cell index, pick order inside the
 * class, image index }, in no particular order.  The reference's output order of an image is: classes by (record[8]
 * descending, record[9] ascending), inside a class by record[10] ascending. */
size_t msnh_hip_yolo_nms_workspace_bytes(int batch, int classes, int cand_cap);
size_t msnh_hip_yolo_nms_pair_workspace_bytes(int batch, int classes, int cand_cap);
int msnh_hip_yolo_nms(int batch, int classes, const float *rows, int cand_cap, const int *cand_cnt, float nms_thresh, float *kept,
                      int kept_cap, int *kept_cnt, void *workspace, size_t workspace_bytes, msnh_stream_t s);

/* msnh_hip_yolo_nms for callers that cannot allocate device memory (code under graph capture, tight serving loops, harnesses that
 * forbid it).  No counterpart in the reference.  Same arguments, results and flags as msnh_hip_yolo_nms called with a workspace, but
 * the workspace is a device array inside the library: msnh_hip_yolo_nms_static_max_bytes() = 4 MiB per GPU the library runs on, held
 * until the process ends.  A geometry whose msnh_hip_yolo_nms_workspace_bytes() exceeds that is refused with an error (YOLOv3 / YOLOv4
 * at 608 x 608 with 80 classes, 22743 candidate slots per image, fit up to batch 45).  The call itself allocates and frees nothing; its one-time set-up per device runs
 * in msnh_hip_init (or in the first call on a device that msnh_hip_init did not select; a failure of that set-up is reported by this
 * call, not by msnh_hip_init).  Every call on a GPU shares that GPU's array, so the library puts the calls on a GPU in order: they
 * are enqueued one at a time (a lock), and a call on another stream than the call before it makes its stream wait, on the device,
 * for that call's end; the host does not block.  Calls from several threads or streams are therefore safe but run one after the
 * other.  The exception is a stream under graph capture: a captured call neither waits for earlier calls nor is waited for
 * (events cannot cross a capture's boundary), so a caller who captures this call keeps the replays of that graph apart from every
 * other use of the entry point on the same GPU. */
size_t msnh_hip_yolo_nms_static_max_bytes(void);
int msnh_hip_yolo_nms_static(int batch, int classes, const float *rows, int cand_cap, const int *cand_cnt, float nms_thresh, float *kept,
                             int kept_cap, int *kept_cnt, msnh_stream_t s);

/* Matrix-core ceiling probe (measurement only, no counterpart in the reference): every SIMD runs `iters` rounds of four independent
 * 32x32x16 float16 MFMAs per wavefront with waves_per_simd (1..8) wavefronts resident, no memory traffic.  Reports the rate
 * achieved (dense TFLOP/s), the shader clock held meanwhile (shader cycles per tick of the 100 MHz constant clock, read by the
 * first wavefront) and the launch's duration.  The rate a fully loaded part sustains, not the published peak at the maximum
 * engine clock, is the practical ceiling of the convolution kernels. */
int msnh_hip_mfma_probe(int waves_per_simd, int iters, double *tflops, double *shader_mhz, double *seconds, msnh_stream_t s);

/* max |x| over the finite elements of an NHWC tensor, combined into *result with an atomic max
 * (caller zeroes *result).  Used once at load time to calibrate the power-of-two activation scales of the
 * float16 plan; no counterpart in the reference. */
int msnh_hip_absmax(int dtype, long long pixels, int c, const void *x, int x_ld, float *result, msnh_stream_t s);

/* Number of elements of an NHWC tensor that are infinite or NaN, added to *result (caller zeroes it).  With msnh_hip_absmax
 * the run-time check of the float16 plan's range: a non-finite element of a float16 activation tensor means an input ran past
 * the headroom of the calibrated scales.  No counterpart in the reference. */
int msnh_hip_count_nonfinite(int dtype, long long pixels, int c, const void *x, int x_ld, unsigned *result, msnh_stream_t s);

#ifdef __cplusplus
}
#endif
#endif
