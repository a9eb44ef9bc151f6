/* TEST INFRASTRUCTURE ONLY -- see msnh_oracle.h.  Plain C restatement of the reference CPU path. */
#include "msnh_oracle.h"
#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* Gemm::cpuIm2colEx, generic branch (src/core/MsnhGemm.cpp:156-292):
 * col[((c*kH+kr)*kW+kc)*outH*outW + oy*outW + ox] = im[c][oy*sH-pH+kr*dH][ox*sW-pW+kc*dW] or 0. */
void msnh_or_im2col(const float *im, int channels, int height, int width, int kH, int kW, int padH, int padW,
                    int strideH, int strideW, int dilH, int dilW, float *col)
{
    const int outH = (height + 2 * padH - (dilH * (kH - 1) + 1)) / strideH + 1;
    const int outW = (width + 2 * padW - (dilW * (kW - 1) + 1)) / strideW + 1;
    for (int c = 0; c < channels; ++c)
        for (int kr = 0; kr < kH; ++kr)
            for (int kc = 0; kc < kW; ++kc)
            {
                float *dst = col + (((size_t)c * kH + kr) * kW + kc) * outH * outW;
                for (int oy = 0; oy < outH; ++oy)
                {
                    const int iy = oy * strideH - padH + kr * dilH;
                    for (int ox = 0; ox < outW; ++ox)
                    {
                        const int ix = ox * strideW - padW + kc * dilW;
                        const int ok = iy >= 0 && iy < height && ix >= 0 && ix < width;
                        dst[oy * outW + ox] = ok ? im[((size_t)c * height + iy) * width + ix] : 0.f;
                    }
                }
            }
}

/* Gemm::cpuGemm(0,0,..,ALPHA=1,..,BETA=1,..) scalar branch -> cpuGemmNN row by row
 * (src/core/MsnhGemm.cpp:888-935, 1071-1208): C[i][j] += A[i][k]*B[k][j], k ascending, float. */
void msnh_or_gemm_nn(int M, int N, int K, const float *A, int lda, const float *B, int ldb, float *C, int ldc)
{
#pragma omp parallel for schedule(static)
    for (int i = 0; i < M; ++i)
        for (int k = 0; k < K; ++k)
        {
            const float a = A[(size_t)i * lda + k];
            const float *b = B + (size_t)k * ldb;
            float *c = C + (size_t)i * ldc;
            for (int j = 0; j < N; ++j)
                c[j] += a * b[j];
        }
}

/* Gemm::cpuGemm(0,1,...) -> cpuGemmNT: C[i][j] += sum_k A[i][k]*B[j][k] (connected layer,
 * src/layers/MsnhConnectedLayer.cpp:187). */
void msnh_or_gemm_nt(int M, int N, int K, const float *A, int lda, const float *B, int ldb, float *C, int ldc)
{
#pragma omp parallel for schedule(static) collapse(2)
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j)
        {
            float sum = 0.f;
            for (int k = 0; k < K; ++k)
                sum += A[(size_t)i * lda + k] * B[(size_t)j * ldb + k];
            C[(size_t)i * ldc + j] += sum;
        }
}

/* Scalar activations (include/Msnhnet/layers/MsnhActivations.h:39-168). */
static float softplus_thr(float x, float thr)
{
    if (x > thr) return x;
    if (x < -thr) return expf(x);
    return logf(expf(x) + 1);
}

float msnh_or_activate(float x, int act, float param)
{
    switch (act)
    {
    case MSNH_OR_ACT_LOGISTIC: return 1.f / (1.f + expf(-x));
    case MSNH_OR_ACT_RELU:     return x * (x > 0);
    case MSNH_OR_ACT_RELU6:    return (x > 0 ? x : 0) > 6 ? 6 : (x > 0 ? x : 0);
    case MSNH_OR_ACT_LEAKY:    return (x > 0) ? x : param * x;
    case MSNH_OR_ACT_SWISH:    return x * (1.f / (1.f + expf(-x)));
    case MSNH_OR_ACT_HARD_SWISH:
    {
        const float t = x + 3.f;                 /* x*relu6Activate(x+3.f)/6.f (MsnhActivations.h:59-62) */
        const float r = (t > 0 ? t : 0) > 6 ? 6 : (t > 0 ? t : 0);
        return x * r / 6.f;
    }
    case MSNH_OR_ACT_MISH:     return x * tanhf(softplus_thr(x, 20.f));
    default:                   return x;
    }
}

void msnh_or_activate_array(float *x, long long n, int act, float param)
{
    if (act == MSNH_OR_ACT_NONE) return;
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < n; ++i)
        x[i] = msnh_or_activate(x[i], act, param);
}

/* Inference batch-norm as the reference evaluates it (src/layers/MsnhConvolutionalLayer.cpp:811-855,
 * src/layers/MsnhBatchNormLayer.cpp:160-200): sqrtVal = sqrt(var+eps) (double sqrt of a float sum,
 * rounded to float), scaleSqrt = g/sqrtVal, meanSqrt = -g*mean/sqrtVal, y = scaleSqrt*x + meanSqrt + b. */
void msnh_or_bn_affine(float *x, int batch, int channels, int hw, const float *scales, const float *biases,
                       const float *mean, const float *var, float eps)
{
    for (int b = 0; b < batch; ++b)
#pragma omp parallel for schedule(static)
        for (int c = 0; c < channels; ++c)
        {
            const float sqrtVal = (float)sqrt(var[c] + eps);
            const float scaleSqrt = scales[c] / sqrtVal;
            const float meanSqrt = -scales[c] * mean[c] / sqrtVal;
            float *p = x + ((size_t)b * channels + c) * hw;
            for (int i = 0; i < hw; ++i)
                p[i] = scaleSqrt * p[i] + meanSqrt + biases[c];
        }
}

/* ConvolutionalLayer::forward (src/layers/MsnhConvolutionalLayer.cpp:553-911): zero fill, per (batch,group)
 * im2col (skipped for 1x1 s1 p0, :743-754) + GEMM M=filters/g N=outH*outW K=channels/g*k*k (:756),
 * then BN or bias (:770-865), then activation (:891-900).  Output dims :388-398. */
void msnh_or_conv(const float *in, int batch, int channels, int height, int width, const float *weights, int filters,
                  int ksize, int stride, int pad, int dilation, int groups, const float *bn4, const float *bias,
                  float eps, int act, float actParam, float *ws, float *out)
{
    const int outH = (height + 2 * pad - (dilation * (ksize - 1) + 1)) / stride + 1;
    const int outW = (width + 2 * pad - (dilation * (ksize - 1) + 1)) / stride + 1;
    const int m = filters / groups;
    const int k = ksize * ksize * channels / groups;
    const int n = outH * outW;
    const size_t nWeights = (size_t)(channels / groups) * filters * ksize * ksize;
    memset(out, 0, sizeof(float) * (size_t)batch * filters * n);
    for (int b = 0; b < batch; ++b)
        for (int g = 0; g < groups; ++g)
        {
            const float *a = weights + (size_t)g * nWeights / groups;
            const float *im = in + ((size_t)b * groups + g) * (channels / groups) * height * width;
            float *c = out + ((size_t)b * groups + g) * n * m;
            const float *bm = im;
            if (!(ksize == 1 && stride == 1 && pad == 0))
            {
                msnh_or_im2col(im, channels / groups, height, width, ksize, ksize, pad, pad, stride, stride,
                               dilation, dilation, ws);
                bm = ws;
            }
            msnh_or_gemm_nn(m, n, k, a, k, bm, n, c, n);
        }
    if (bn4)
        msnh_or_bn_affine(out, batch, filters, n, bn4, bn4 + filters, bn4 + 2 * filters, bn4 + 3 * filters, eps);
    else if (bias)
        for (int b = 0; b < batch; ++b)
            for (int f = 0; f < filters; ++f)
            {
                float *p = out + ((size_t)b * filters + f) * n;
                for (int i = 0; i < n; ++i)
                    p[i] += bias[f];
            }
    msnh_or_activate_array(out, (long long)batch * filters * n, act, actParam);
}

/* BatchNormLayer::forward (src/layers/MsnhBatchNormLayer.cpp:54-254). */
void msnh_or_batchnorm(const float *in, int batch, int channels, int hw, const float *bn4, float eps, int act,
                       float actParam, float *out)
{
    if (out != in)
        memcpy(out, in, sizeof(float) * (size_t)batch * channels * hw);
    msnh_or_bn_affine(out, batch, channels, hw, bn4, bn4 + channels, bn4 + 2 * channels, bn4 + 3 * channels, eps);
    msnh_or_activate_array(out, (long long)batch * channels * hw, act, actParam);
}

/* MaxPoolLayer::forward scalar branch (src/layers/MsnhMaxPoolLayer.cpp:293-345): padding = -FLT_MAX. */
void msnh_or_maxpool(const float *in, int batch, int channels, int height, int width, int ksize, int stride, int pad,
                     int outH, int outW, float *out)
{
#pragma omp parallel for schedule(static) collapse(2)
    for (int b = 0; b < batch; ++b)
        for (int c = 0; c < channels; ++c)
            for (int i = 0; i < outH; ++i)
                for (int j = 0; j < outW; ++j)
                {
                    float mx = -FLT_MAX;
                    for (int n = 0; n < ksize; ++n)
                        for (int m = 0; m < ksize; ++m)
                        {
                            const int y = -pad + i * stride + n;
                            const int x = -pad + j * stride + m;
                            const int ok = y >= 0 && y < height && x >= 0 && x < width;
                            const float v = ok ? in[(((size_t)b * channels + c) * height + y) * width + x] : -FLT_MAX;
                            mx = (v > mx) ? v : mx;
                        }
                    out[(((size_t)b * channels + c) * outH + i) * outW + j] = mx;
                }
}

/* LocalAvgPoolLayer::forward (src/layers/MsnhLocalAvgPoolLayer.cpp:286-344): mean over the valid
 * window elements only, accumulated in row-major window order, divided by their count. */
void msnh_or_avgpool(const float *in, int batch, int channels, int height, int width, int ksize, int stride, int pad,
                     int outH, int outW, float *out)
{
    for (int b = 0; b < batch; ++b)
        for (int c = 0; c < channels; ++c)
            for (int i = 0; i < outH; ++i)
                for (int j = 0; j < outW; ++j)
                {
                    float avg = 0;
                    int counter = 0;
                    for (int n = 0; n < ksize; ++n)
                        for (int m = 0; m < ksize; ++m)
                        {
                            const int y = -pad + i * stride + n;
                            const int x = -pad + j * stride + m;
                            if (y >= 0 && y < height && x >= 0 && x < width)
                            {
                                counter++;
                                avg += in[(((size_t)b * channels + c) * height + y) * width + x];
                            }
                        }
                    out[(((size_t)b * channels + c) * outH + i) * outW + j] = avg / counter;
                }
}

/* ConnectedLayer::forward without batch-norm (src/layers/MsnhConnectedLayer.cpp:176-240). */
void msnh_or_connected(const float *in, int batch, int inputs, int outputs, const float *weights, const float *bias,
                       int act, float actParam, float *out)
{
    memset(out, 0, sizeof(float) * (size_t)batch * outputs);
    msnh_or_gemm_nt(batch, outputs, inputs, in, inputs, weights, inputs, out, outputs);
    if (bias)
        for (int b = 0; b < batch; ++b)
            for (int o = 0; o < outputs; ++o)
                out[(size_t)b * outputs + o] += bias[o];
    msnh_or_activate_array(out, (long long)batch * outputs, act, actParam);
}

/* Blas::cpuUpSample (src/core/MsnhBlas.cpp:2354-2398): out[c][j][i] = scale*in[c][j/sy][i/sx]. */
void msnh_or_upsample(const float *in, int batch, int channels, int height, int width, int strideX, int strideY,
                      float scale, float *out)
{
    const int oh = height * strideY, ow = width * strideX;
    for (int b = 0; b < batch; ++b)
        for (int k = 0; k < channels; ++k)
            for (int j = 0; j < oh; ++j)
                for (int i = 0; i < ow; ++i)
                    out[(((size_t)b * channels + k) * oh + j) * ow + i] =
                        scale * in[(((size_t)b * channels + k) * height + j / strideY) * width + i / strideX];
}

/* Blas::cpuAxpy with unit strides (src/core/MsnhBlas.cpp:6-150): y += alpha*x. */
void msnh_or_axpy(long long n, float alpha, const float *x, float *y)
{
    for (long long i = 0; i < n; ++i)
        y[i] += alpha * x[i];
}

/* YoloLayer::forward (src/layers/MsnhYoloLayer.cpp:61-142, helpers :217-296), in place.  Per anchor n:
 *   yolov3 / yolov4 (version 3, 4): plane0 (sigmoid+col)*ratio, plane1 (sigmoid+row)*ratio, plane2 aw*exp, plane3 ah*exp;
 *   yolov5 (version 5): plane0 (2*sigmoid-0.5+col)*ratio, plane1 likewise with row, planes 2,3 a*powf(2*sigmoid, 2);
 *   planes 4.. sigmoid in both. */
void msnh_or_yolo_decode(float *data, int batch, int width, int height, int classNum, const float *anchors6, float ratio,
                         int version)
{
    const int hw = width * height;
    const int per = 5 + classNum;
    for (int b = 0; b < batch; ++b)
        for (int n = 0; n < 3; ++n)
        {
            float *p = data + ((size_t)b * 3 + n) * per * hw;
            if (version == 5)
            {
                for (int i = 0; i < hw; ++i)
                    p[i] = (2.f / (1.f + expf(-p[i])) - 0.5f + i % width) * ratio;
                p += hw;
                for (int i = 0; i < hw; ++i)
                    p[i] = (2.f / (1.f + expf(-p[i])) - 0.5f + i / width) * ratio;
                p += hw;
                for (int i = 0; i < hw; ++i)
                    p[i] = anchors6[n % 3 * 2] * powf(2.f / (1.f + expf(-p[i])), 2.f);
                p += hw;
                for (int i = 0; i < hw; ++i)
                    p[i] = anchors6[n % 3 * 2 + 1] * powf(2.f / (1.f + expf(-p[i])), 2.f);
                p += hw;
            }
            else
            {
                for (int i = 0; i < hw; ++i)
                    p[i] = (1.f / (1.f + expf(-p[i])) + i % width) * ratio;
                p += hw;
                for (int i = 0; i < hw; ++i)
                    p[i] = (1.f / (1.f + expf(-p[i])) + i / width) * ratio;
                p += hw;
                for (int i = 0; i < hw; ++i)
                    p[i] = anchors6[n % 3 * 2] * expf(p[i]);
                p += hw;
                for (int i = 0; i < hw; ++i)
                    p[i] = anchors6[n % 3 * 2 + 1] * expf(p[i]);
                p += hw;
            }
            for (long long i = 0; i < (long long)hw * (1 + classNum); ++i)
                p[i] = 1.f / (1.f + expf(-p[i]));
        }
}

/* PaddingLayer::forward (src/layers/MsnhPaddingLayer.cpp:143-177): constant border around every channel plane. */
void msnh_or_pad(const float *in, int batch, int channels, int height, int width, int top, int down, int left, int right,
                 float value, float *out)
{
    const int oh = height + top + down, ow = width + left + right;
    for (int i = 0; i < batch; ++i)
        for (int j = 0; j < channels; ++j)
            for (int m = 0; m < oh; ++m)
                for (int n = 0; n < ow; ++n)
                {
                    float val;
                    if (m < top || m >= height + top) val = value;
                    else if (n < left || n >= width + left) val = value;
                    else val = in[(((size_t)i * channels + j) * height + (m - top)) * width + (n - left)];
                    out[(((size_t)i * channels + j) * oh + m) * ow + n] = val;
                }
}

/* SliceLayer::forward (src/layers/MsnhSliceLayer.cpp:120-147): out[c][h][w] = in[c*step0+start0][h*step1+start1][w*step2+start2],
 * output extents ceil((extent - start) / step) (ctor, :28-48). */
void msnh_or_slice(const float *in, int batch, int channels, int height, int width, int start0, int step0, int start1, int step1,
                   int start2, int step2, float *out)
{
    const int oc = (channels - start0) / step0 + ((channels - start0) % step0 ? 1 : 0);
    const int oh = (height - start1) / step1 + ((height - start1) % step1 ? 1 : 0);
    const int ow = (width - start2) / step2 + ((width - start2) % step2 ? 1 : 0);
    for (int b = 0; b < batch; ++b)
        for (int c = 0; c < oc; ++c)
            for (int h = 0; h < oh; ++h)
                for (int w = 0; w < ow; ++w)
                    out[(((size_t)b * oc + c) * oh + h) * ow + w] =
                        in[(((size_t)b * channels + c * step0 + start0) * height + h * step1 + start1) * width + w * step2 + start2];
}

/* Blas::cpuBilinearResize (src/core/MsnhBlas.cpp:2400-2465). */
void msnh_or_bilinear(const float *in, int batch, int channels, int height, int width, int outH, int outW, int alignCorners,
                      float *out)
{
    const float rH = alignCorners == 0 ? 1.0f * height / outH : 1.0f * (height - 1) / (outH - 1);
    const float rW = alignCorners == 0 ? 1.0f * width / outW : 1.0f * (width - 1) / (outW - 1);
    const size_t inSize = (size_t)width * height, outSize = (size_t)outW * outH;
    for (size_t i = 0; i < outSize; ++i)
    {
        const int h2 = (int)(i / outW), w2 = (int)(i % outW);
        float h1r, w1r;
        if (alignCorners == 0)
        {
            const float ih = rH * (h2 + 0.5f) - 0.5f;
            const float iw = rW * (w2 + 0.5f) - 0.5f;
            h1r = ih < 0 ? 0 : ih;
            w1r = iw < 0 ? 0 : iw;
        }
        else
        {
            h1r = rH * h2;
            w1r = rW * w2;
        }
        const int h1 = (int)h1r, w1 = (int)w1r;
        const int h1p = h1 < height - 1 ? 1 : 0, w1p = w1 < width - 1 ? 1 : 0;
        const float h1L = h1r - h1, h0L = 1.0f - h1L, w1L = w1r - w1, w0L = 1.0f - w1L;
        const float *ip = in + (size_t)h1 * width + w1;
        for (int c = 0; c < channels * batch; ++c)
        {
            const float *t = ip + c * inSize;
            out[i + c * outSize] = h0L * (w0L * t[0] + w1L * t[w1p]) + h1L * (w0L * t[h1p * width] + w1L * t[h1p * width + w1p]);
        }
    }
}

/* SoftMaxLayer::forward with groups == 1 (src/layers/MsnhSoftMaxLayer.cpp:60-93): Blas::softmax over all inputNum values
 * of each image, scalar path (src/core/MsnhBlas.cpp:2076-2110): e = exp(x/T - max/T) in double, rounded to float. */
void msnh_or_softmax(const float *in, int batch, int num, float temperature, float *out)
{
    for (int b = 0; b < batch; ++b)
    {
        const float *x = in + (size_t)b * num;
        float *y = out + (size_t)b * num;
        float largest = -FLT_MAX, sum = 0;
        for (int i = 0; i < num; ++i)
            if (x[i] > largest) largest = x[i];
        for (int i = 0; i < num; ++i)
        {
            const float e = (float)exp(x[i] / temperature - largest / temperature);
            sum += e;
            y[i] = e;
        }
        for (int i = 0; i < num; ++i)
            y[i] /= sum;
    }
}

/* GlobalAvgPoolLayer::forward (src/layers/MsnhGlobalAvgPoolLayer.cpp:152-168): running float sum over the plane, / (h*w). */
void msnh_or_global_avgpool(const float *in, int batch, int channels, int hw, float *out)
{
    for (int b = 0; b < batch; ++b)
        for (int k = 0; k < channels; ++k)
        {
            float acc = 0;
            for (int i = 0; i < hw; ++i)
                acc += in[((size_t)b * channels + k) * hw + i];
            out[(size_t)b * channels + k] = acc / hw;
        }
}

/* DeConvolutionalLayer::forward, groups == 1 (src/layers/MsnhDeConvolutionalLayer.cpp:140-200): per image
 * col[m][n] = sum_ic W[ic][m] * in[ic][n]  (cpuGemm with A transposed; m = (oc*k + ky)*k + kx, n = pixel), then
 * Gemm::cpuCol2Im (src/core/MsnhGemm.cpp:115-154) accumulates col into the zero-filled output, then bias, activation.
 * weights: [channels][filters][k][k]. */
void msnh_or_deconv(const float *in, int batch, int channels, int height, int width, const float *weights, int filters, int ksize,
                    int stride, int pad, const float *bias, int act, float actParam, float *out)
{
    const int oh = (height - 1) * stride - 2 * pad + ksize, ow = (width - 1) * stride - 2 * pad + ksize;
    const int m = ksize * ksize * filters, n = height * width;
    float *col = (float *)malloc((size_t)m * n * sizeof(float));
    for (int b = 0; b < batch; ++b)
    {
        const float *x = in + (size_t)b * channels * n;
        float *y = out + (size_t)b * filters * oh * ow;
        memset(y, 0, (size_t)filters * oh * ow * sizeof(float));
#pragma omp parallel for schedule(static)
        for (int i = 0; i < m; ++i)
            for (int j = 0; j < n; ++j)
            {
                float sum = 0;
                for (int k = 0; k < channels; ++k)
                    sum += weights[(size_t)k * m + i] * x[(size_t)k * n + j];
                col[(size_t)i * n + j] = sum;
            }
        for (int c = 0; c < m; ++c)
        {
            const int wOff = c % ksize, hOff = (c / ksize) % ksize, cIm = c / ksize / ksize;
            for (int h = 0; h < height; ++h)
                for (int w = 0; w < width; ++w)
                {
                    const int r = hOff + h * stride - pad, q = wOff + w * stride - pad;
                    if (r < 0 || q < 0 || r >= oh || q >= ow) continue;
                    y[q + (size_t)ow * (r + (size_t)oh * cIm)] += col[((size_t)c * height + h) * width + w];
                }
        }
        for (int f = 0; f < filters; ++f)
            for (int i = 0; i < oh * ow; ++i)
            {
                float v = y[(size_t)f * oh * ow + i];
                if (bias) v += bias[f];
                y[(size_t)f * oh * ow + i] = msnh_or_activate(v, act, actParam);
            }
    }
    free(col);
}

/* Box::iou (include/Msnhnet/utils/MsnhTypes.h:104-140), including its +1 pixel convention. */
float msnh_or_iou(const float *a, const float *b)
{
    const float ax1 = a[0] - a[2] / 2.f, ax2 = a[0] + a[2] / 2.f, ay1 = a[1] - a[3] / 2.f, ay2 = a[1] + a[3] / 2.f;
    const float bx1 = b[0] - b[2] / 2.f, bx2 = b[0] + b[2] / 2.f, by1 = b[1] - b[3] / 2.f, by2 = b[1] + b[3] / 2.f;
    /* std::max(a,b) = (a<b)?b:a ; std::min(a,b) = (b<a)?b:a  (NaN behaviour preserved) */
    const float ix1 = (ax1 < bx1) ? bx1 : ax1;
    const float iy1 = (ay1 < by1) ? by1 : ay1;
    const float ix2 = (bx2 < ax2) ? bx2 : ax2;
    const float iy2 = (by2 < ay2) ? by2 : ay2;
    const float iw = ix2 - ix1 + 1;
    const float ih = iy2 - iy1 + 1;
    const float inter = (iw < 0 ? 0 : iw) * (ih < 0 ? 0 : ih);
    const float a1 = (ax2 - ax1 + 1) * (ay2 - ay1 + 1);
    const float a2 = (bx2 - bx1 + 1) * (by2 - by1 + 1);
    return 1.f * inter / (a1 + a2 - inter);
}

typedef struct { float x, y, w, h, conf, best; int cls; float key; int order; } or_box;

static int cmp_desc(const void *pa, const void *pb)
{
    const or_box *a = (const or_box *)pa, *b = (const or_box *)pb;
    /* the reference sorts indices with the unstable std::sort on key ">" (include/Msnhnet/utils/MsnhExVector.h:58-74);
     * ties are broken here by original order, callers compare box sets order-insensitively. */
    if (a->key > b->key) return -1;
    if (a->key < b->key) return 1;
    return (a->order > b->order) - (a->order < b->order);
}

/* YoloOutLayer::forward for one image + YoloOutLayer::nms (src/layers/MsnhYoloOutLayer.cpp:79-203, 381-461):
 * heads are visited in the given order, each transposed to [anchor][pixel][5+classes]; keep obj > confThresh;
 * best class = first maximum; stable order by obj*bestCls descending; per class (in first-appearance order)
 * greedy NMS picking the highest obj (first on ties) and erasing iou > nmsThresh; single-box classes pass. */
long long msnh_or_yolo_out(const float *const *heads, const int *hw, int nHeads, int classNum, float confThresh,
                           float nmsThresh, float *boxes, long long capBoxes)
{
    const int per = 5 + classNum;
    long long total = 0;
    for (int i = 0; i < nHeads; ++i) total += 3LL * hw[i];
    or_box *cand = (or_box *)malloc(sizeof(or_box) * (size_t)(total > 0 ? total : 1));
    long long n = 0;
    for (int i = 0; i < nHeads; ++i)
        for (int k = 0; k < 3; ++k)
            for (int p = 0; p < hw[i]; ++p)
            {
                const float *base = heads[i] + (size_t)k * per * hw[i] + p;   /* element m at base[m*hw] */
                const float obj = base[4 * (size_t)hw[i]];
                if (obj > confThresh)
                {
                    or_box q;
                    q.x = base[0]; q.y = base[(size_t)hw[i]]; q.w = base[2 * (size_t)hw[i]]; q.h = base[3 * (size_t)hw[i]];
                    q.conf = obj;
                    int best = 0;
                    float bv = base[5 * (size_t)hw[i]];
                    for (int m = 1; m < classNum; ++m)
                    {
                        const float v = base[(size_t)(5 + m) * hw[i]];
                        if (bv < v) { bv = v; best = m; }      /* std::max_element: first maximum */
                    }
                    q.best = bv; q.cls = best; q.key = q.conf * q.best; q.order = (int)n;
                    cand[n++] = q;
                }
            }
    if (n > 0) qsort(cand, (size_t)n, sizeof(or_box), cmp_desc);

    long long nOut = 0;
    char *done = (char *)calloc((size_t)(n > 0 ? n : 1), 1);       /* class already processed */
    or_box *cls = (or_box *)malloc(sizeof(or_box) * (size_t)(n > 0 ? n : 1));
    for (long long i = 0; i < n; ++i)
    {
        if (done[i]) continue;
        const int c = cand[i].cls;
        long long m = 0;
        for (long long j = i; j < n; ++j)
            if (cand[j].cls == c) { cls[m++] = cand[j]; done[j] = 1; }
        if (m == 1)
        {
            if (nOut < capBoxes && boxes)
            {
                float *o = boxes + 7 * nOut;
                o[0] = cls[0].x; o[1] = cls[0].y; o[2] = cls[0].w; o[3] = cls[0].h; o[4] = cls[0].conf; o[5] = cls[0].best; o[6] = (float)c;
            }
            nOut++;
            continue;
        }
        while (m > 0)
        {
            long long bi = 0;
            float bc = -FLT_MAX;
            for (long long j = 0; j < m; ++j)
                if (cls[j].conf > bc) { bi = j; bc = cls[j].conf; }
            const or_box best = cls[bi];
            if (nOut < capBoxes && boxes)
            {
                float *o = boxes + 7 * nOut;
                o[0] = best.x; o[1] = best.y; o[2] = best.w; o[3] = best.h; o[4] = best.conf; o[5] = best.best; o[6] = (float)c;
            }
            nOut++;
            memmove(cls + bi, cls + bi + 1, sizeof(or_box) * (size_t)(m - bi - 1));
            m--;
            long long w = 0;
            for (long long j = 0; j < m; ++j)
            {
                const float iou = msnh_or_iou(&cls[j].x, &best.x);
                if (!(iou > nmsThresh)) cls[w++] = cls[j];
            }
            m = w;
        }
    }
    free(cls); free(done); free(cand);
    return nOut;
}

/* ---- pre / post-processing around the graph ------------------------------------------------------------------- */

/* CVUtil::getPaddingZeroF32C3 for a 3-channel 8-bit image (src/utils/MsnhCVUtil.cpp:203-261):
 *   - pad the shorter side to a square with (127,127,127): top/left = diff/2, bottom/right = diff - diff/2
 *     (:216-225; MatOp::copyMakeBorder, include/Msnhnet/cv/MsnhCVMatOp.h:18-54);
 *   - MatOp::resize to (netW, netH), bilinear, MAT_RGB_U8 branch (src/cv/MsnhCVMatOp.cpp:142-160, 404-437): no resize
 *     when the size already matches (:152-156); source coordinate (i+0.5)*f-0.5 clamped below at 0 only; second
 *     sample index min(i0+1, n-1); weights (i1 - s) and (s - i0), which sum to 0 where i1 == i0 (the reference's
 *     behaviour when enlarging: the last rows/columns come out 0); float arithmetic in the order written there,
 *     truncation to uint16 and a clamp at 255;
 *   - cvtColor RGB2BGR when asked (:232-233);
 *   - v/255 or (v-127.5)/127.5, HWC -> CHW (:243-257). */
void msnh_or_letterbox_u8(const unsigned char *img, int width, int height, int netW, int netH, int halfInit,
                          int shuffleRGB, float *out)
{
    const int diff = abs(width - height);
    const int top = width > height ? diff / 2 : 0;
    const int left = width < height ? diff / 2 : 0;
    const int S = width > height ? width : height;
    unsigned char *sq = (unsigned char *)malloc((size_t)S * S * 3);
    memset(sq, 127, (size_t)S * S * 3);
    for (int y = 0; y < height; ++y)
        memcpy(sq + ((size_t)(y + top) * S + left) * 3, img + (size_t)y * width * 3, (size_t)width * 3);

    unsigned char *rs = sq;
    if (!(netW == S && netH == S))
    {
        rs = (unsigned char *)calloc((size_t)netW * netH * 3, 1);
        const float fx = 1.f * S / netW;
        const float fy = 1.f * S / netH;
        for (int i = 0; i < netH; ++i)
        {
            float sh = (i + 0.5f) * fy - 0.5f;
            sh = sh < 0 ? 0 : sh;
            const int h0 = (int)sh;
            const int h1 = h0 + 1 < S - 1 ? h0 + 1 : S - 1;
            for (int j = 0; j < netW; ++j)
            {
                float sw = (j + 0.5f) * fx - 0.5f;
                sw = sw < 0 ? 0 : sw;
                const int w0 = (int)sw;
                const int w1 = w0 + 1 < S - 1 ? w0 + 1 : S - 1;
                for (int k = 0; k < 3; ++k)
                {
                    const float v = (h1 - sh) * ((w1 - sw) * sq[3 * ((size_t)h0 * S + w0) + k] + (sw - w0) * sq[3 * ((size_t)h0 * S + w1) + k]) +
                                    (sh - h0) * ((w1 - sw) * sq[3 * ((size_t)h1 * S + w0) + k] + (sw - w0) * sq[3 * ((size_t)h1 * S + w1) + k]);
                    const unsigned short r = (unsigned short)v;
                    rs[3 * ((size_t)i * netW + j) + k] = (unsigned char)(r > 255 ? 255 : r);
                }
            }
        }
    }
    for (int y = 0; y < netH; ++y)
        for (int k = 0; k < 3; ++k)
            for (int x = 0; x < netW; ++x)
            {
                const unsigned char u = rs[3 * ((size_t)y * netW + x) + (shuffleRGB ? 2 - k : k)];
                out[(size_t)k * netW * netH + (size_t)y * netW + x] = halfInit ? (u - 127.5f) / 127.5f : u / 255.0f;
            }
    if (rs != sq) free(rs);
    free(sq);
}

/* The plain-resize pre-processing variants of CVUtil for a 3-channel 8-bit image (src/utils/MsnhCVUtil.cpp):
 *   kind 0  getImgDataF32C3, halfInit 0 (:91-138)      u / 255
 *   kind 1  getImgDataF32C3, halfInit 1                 (u - 127.5) / 127.5
 *   kind 2  getGoogLenetF32C3 (:146-195)                u / 255 * (std_k / 0.5) + (mean_k - 0.5) / 0.5  with the ImageNet constants written there
 *   kind 3  getTransformedF32C3 (:269-318)              (u / 255 - mean[k]) / std[k]
 *   kind 4  getCaffeModeF32C3 (:326-375)                u - {123.68, 116.779, 103.939}[k]
 * all after MatOp::resize to (netW, netH) (src/cv/MsnhCVMatOp.cpp:142-160, 404-437: fx = srcW / dstW, fy = srcH / dstH, see
 * msnh_or_letterbox_u8 for the arithmetic; no resize when the size already matches) and the optional RGB2BGR swap; HWC -> CHW. */
void msnh_or_preproc_u8(const unsigned char *img, int width, int height, int netW, int netH, int kind, const float *mean,
                        const float *stdv, int shuffleRGB, float *out)
{
    const unsigned char *rs = img;
    unsigned char *tmp = NULL;
    if (!(netW == width && netH == height))
    {
        tmp = (unsigned char *)calloc((size_t)netW * netH * 3, 1);
        const float fx = 1.f * width / netW;
        const float fy = 1.f * height / netH;
        for (int i = 0; i < netH; ++i)
        {
            float sh = (i + 0.5f) * fy - 0.5f;
            sh = sh < 0 ? 0 : sh;
            const int h0 = (int)sh;
            const int h1 = h0 + 1 < height - 1 ? h0 + 1 : height - 1;
            for (int j = 0; j < netW; ++j)
            {
                float sw = (j + 0.5f) * fx - 0.5f;
                sw = sw < 0 ? 0 : sw;
                const int w0 = (int)sw;
                const int w1 = w0 + 1 < width - 1 ? w0 + 1 : width - 1;
                for (int k = 0; k < 3; ++k)
                {
                    const float v = (h1 - sh) * ((w1 - sw) * img[3 * ((size_t)h0 * width + w0) + k] + (sw - w0) * img[3 * ((size_t)h0 * width + w1) + k]) +
                                    (sh - h0) * ((w1 - sw) * img[3 * ((size_t)h1 * width + w0) + k] + (sw - w0) * img[3 * ((size_t)h1 * width + w1) + k]);
                    const unsigned short r = (unsigned short)v;
                    tmp[3 * ((size_t)i * netW + j) + k] = (unsigned char)(r > 255 ? 255 : r);
                }
            }
        }
        rs = tmp;
    }
    static const float gStd[3] = {0.229f, 0.224f, 0.225f}, gMean[3] = {0.485f, 0.456f, 0.406f};
    static const float caffe[3] = {123.68f, 116.779f, 103.939f};
    for (int y = 0; y < netH; ++y)
        for (int k = 0; k < 3; ++k)
            for (int x = 0; x < netW; ++x)
            {
                const unsigned char u = rs[3 * ((size_t)y * netW + x) + (shuffleRGB ? 2 - k : k)];
                float v;
                switch (kind)
                {
                case 1:  v = (u - 127.5f) / 127.5f; break;
                case 2:  v = u / 255.0f * (gStd[k] / 0.5f) + (gMean[k] - 0.5f) / 0.5f; break;
                case 3:  v = ((u / 255.0f) - mean[k]) / stdv[k]; break;
                case 4:  v = (u) - caffe[k]; break;
                default: v = u / 255.0f; break;
                }
                out[(size_t)k * netW * netH + (size_t)y * netW + x] = v;
            }
    free(tmp);
}

/* YoloOutLayer::bboxResize2Org (src/layers/MsnhYoloOutLayer.cpp:321-361): undo the letterbox */
void msnh_or_bbox_resize2org(float *b, int curW, int curH, int orgW, int orgH)
{
    if (orgW > orgH)
    {
        const float scaledRatio = 1.0f * curW / orgW;
        const int padUp = (int)((curH - orgH * scaledRatio) / 2);
        b[0] = b[0] / scaledRatio;
        b[2] = b[2] / scaledRatio;
        b[1] = (b[1] - padUp) / scaledRatio;
        b[3] = b[3] / scaledRatio;
    }
    else
    {
        const float scaledRatio = 1.0f * curH / orgH;
        const int padLeft = (int)((curW - orgW * scaledRatio) / 2);
        b[0] = (b[0] - padLeft) / scaledRatio;
        b[2] = b[2] / scaledRatio;
        b[1] = b[1] / scaledRatio;
        b[3] = b[3] / scaledRatio;
    }
}

/* YoloOutLayer::bboxResize2OrgNoPad (:363-379): undo a plain (aspect-changing) resize */
void msnh_or_bbox_resize2org_nopad(float *b, int curW, int curH, int orgW, int orgH)
{
    const float scaledRatioW = 1.0f * curW / orgW;
    const float scaledRatioH = 1.0f * curH / orgH;
    b[0] = b[0] / scaledRatioW;
    b[2] = b[2] / scaledRatioW;
    b[1] = b[1] / scaledRatioH;
    b[3] = b[3] / scaledRatioH;
}
