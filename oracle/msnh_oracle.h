/* TEST INFRASTRUCTURE ONLY -- a plain-C restatement of the reference's CPU algorithm for the
 * convolutional hot path.  Only tests, the smoke check and the CPU-baseline leg of the benchmark may
 * link or load it; the product never does.
 *
 * Tensors are NCHW float32 exactly as in the reference.  Every function cites the reference code it
 * restates.  How each function is pinned (see tests/test_oracle_*.py):
 *   - all of them: against the compiled reference (oracle/_ref) on seeded inputs, layer by layer;
 *   - conv/im2col/gemm: brute-force double-precision cross-correlation, identity kernels, 1x1 == GEMM;
 *   - batchnorm/activations: closed forms and special values;
 *   - maxpool/avgpool/upsample: brute force and index formula;
 *   - yolo decode / iou / nms: closed form per element, hand-built box sets.
 */
#ifndef MSNH_ORACLE_H
#define MSNH_ORACLE_H
#ifdef __cplusplus
extern "C" {
#endif

/* values of the reference's ActivationType (include/Msnhnet/config/MsnhnetCfg.h:95-120) */
enum { MSNH_OR_ACT_LOGISTIC = 0, MSNH_OR_ACT_RELU = 1, MSNH_OR_ACT_RELU6 = 2, MSNH_OR_ACT_LEAKY = 8,
       MSNH_OR_ACT_SWISH = 16, MSNH_OR_ACT_HARD_SWISH = 17, MSNH_OR_ACT_MISH = 18, MSNH_OR_ACT_NONE = 22 };

void  msnh_or_im2col(const float *im, int channels, int height, int width, int kH, int kW, int padH, int padW,
                     int strideH, int strideW, int dilH, int dilW, float *col);
void  msnh_or_gemm_nn(int M, int N, int K, const float *A, int lda, const float *B, int ldb, float *C, int ldc);
void  msnh_or_gemm_nt(int M, int N, int K, const float *A, int lda, const float *B, int ldb, float *C, int ldc);
float msnh_or_activate(float x, int act, float param);
void  msnh_or_activate_array(float *x, long long n, int act, float param);
void  msnh_or_bn_affine(float *x, int batch, int channels, int hw, const float *scales, const float *biases,
                        const float *mean, const float *var, float eps);
/* bn4 = {scales,biases,rollMean,rollVariance} concatenated (each `filters` long) or NULL; bias NULL = none.
 * ws must hold (channels/groups)*k*k*outH*outW floats. */
void  msnh_or_conv(const float *in, int batch, int channels, int height, int width, const float *weights, int filters,
                   int ksize, int stride, int pad, int dilation, int groups, const float *bn4, const float *bias,
                   float eps, int act, float actParam, float *ws, float *out);
void  msnh_or_batchnorm(const float *in, int batch, int channels, int hw, const float *bn4, float eps, int act,
                        float actParam, float *out);
void  msnh_or_maxpool(const float *in, int batch, int channels, int height, int width, int ksize, int stride, int pad,
                      int outH, int outW, float *out);
void  msnh_or_avgpool(const float *in, int batch, int channels, int height, int width, int ksize, int stride, int pad,
                      int outH, int outW, float *out);
void  msnh_or_connected(const float *in, int batch, int inputs, int outputs, const float *weights, const float *bias,
                        int act, float actParam, float *out);
void  msnh_or_upsample(const float *in, int batch, int channels, int height, int width, int strideX, int strideY,
                       float scale, float *out);
void  msnh_or_axpy(long long n, float alpha, const float *x, float *y);
/* version 3 / 4: yolov3 and yolov4 decoding; 5: yolov5 */
void  msnh_or_yolo_decode(float *data, int batch, int width, int height, int classNum, const float *anchors6, float ratio,
                          int version);
void  msnh_or_pad(const float *in, int batch, int channels, int height, int width, int top, int down, int left, int right,
                  float value, float *out);
void  msnh_or_slice(const float *in, int batch, int channels, int height, int width, int start0, int step0, int start1, int step1,
                    int start2, int step2, float *out);
void  msnh_or_deconv(const float *in, int batch, int channels, int height, int width, const float *weights, int filters, int ksize,
                     int stride, int pad, const float *bias, int act, float actParam, float *out);
void  msnh_or_softmax(const float *in, int batch, int num, float temperature, float *out);
void  msnh_or_global_avgpool(const float *in, int batch, int channels, int hw, float *out);
void  msnh_or_bilinear(const float *in, int batch, int channels, int height, int width, int outH, int outW, int alignCorners,
                       float *out);
float msnh_or_iou(const float *xywh1, const float *xywh2);
/* One image.  heads[i] points at a decoded head [3*(5+classes)][hw[i]]; boxes out as rows of
 * 7 floats (x y w h conf bestClsConf bestClsIdx).  Returns the box count (may exceed capBoxes). */
long long msnh_or_yolo_out(const float *const *heads, const int *hw, int nHeads, int classNum, float confThresh,
                           float nmsThresh, float *boxes, long long capBoxes);

/* The step either side of the graph.
 * Letterbox of one 3-channel 8-bit HWC image to the network input: pad to a square with 127, bilinear resize,
 * optional R<->B swap, scale to [0,1] (half_init 0) or [-1,1] (half_init 1), HWC -> CHW float. */
void  msnh_or_letterbox_u8(const unsigned char *img, int width, int height, int netW, int netH, int halfInit,
                           int shuffleRGB, float *out);
void  msnh_or_preproc_u8(const unsigned char *img, int width, int height, int netW, int netH, int kind, const float *mean,
                          const float *stdv, int shuffleRGB, float *out);
/* Box (x y w h, centre form, network-input pixels) back to the original image; in place. */
void  msnh_or_bbox_resize2org(float *xywh, int curW, int curH, int orgW, int orgH);
void  msnh_or_bbox_resize2org_nopad(float *xywh, int curW, int curH, int orgW, int orgH);

#ifdef __cplusplus
}
#endif
#endif
