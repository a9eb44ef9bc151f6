/*
 * msnhnet_c.h -- C ABI of the host library `libMsnhnet.so` (NetBuilder build / load / run).
 *
 * Part 1 keeps the names and argument meaning of the reference's C facade (src/c_api/MsnhnetLib.h:39-61), which
 * drives one process-wide network.  Part 2 is a handle-based variant of the same calls (several networks,
 * batches, per-layer dumps, device-resident inputs) used by the tests and the benchmark.
 * All functions return 1 on success and -1 on failure like the reference's (MsnhnetLib.cpp:10-35) unless stated;
 * the message of the last failure is kept in static storage (the reference returns a pointer into a destroyed
 * local, src/c_api/MsnhnetLib.cpp:29-31).
 */
#ifndef MSNHNET_C_H
#define MSNHNET_C_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MSNHNET_MAX_BBOX 1024          /* MaxBBoxNum, src/c_api/MsnhnetLib.h:9 */

typedef struct BBox                    /* src/c_api/MsnhnetLib.h:22-32 */
{
    float    x, y, w, h;
    float    conf;
    float    bestClsConf;
    uint32_t bestClsIdx;
    float    angle;
} BBox;

typedef struct BBoxContainer           /* src/c_api/MsnhnetLib.h:34-37 */
{
    BBox boxes[MSNHNET_MAX_BBOX];
} BBoxContainer;

/* PredDataType, src/c_api/MsnhnetLib.h:11-20 */
enum PredDataType
{
    PRE_DATA_NONE = 0,
    PRE_DATA_FC32_C1,
    PRE_DATA_FC32_C3,
    PRE_DATA_GOOGLENET_FC3,
    PRE_DATA_PADDING_ZERO_FC3,
    PRE_DATA_TRANSFORMED_FC3,
    PRE_DATA_CAFFE_FC3
};

/* ---- part 1: the reference facade -------------------------------------------------------------------------------- */
int initMsnhnet(void);                                                                  /* MsnhnetLib.h:39 */
int buildMsnhnet(char **msg, const char *msnhnet, const char *msnhbin, int useFp16, int useCudaOnly);   /* :40 */
/* data = one CHW float image (or batch*CHW when the graph's batch > 1); runGPU must be non-zero: the CPU path
 * does not exist in this build and runGPU == 0 fails with "Gpu mode , can not run with cpu".            :49 */
int runClassifyNoPred(char **msg, const float *data, const int len, int *bestIndex, int runGPU);
/* Same contract for detection networks; fills at most MSNHNET_MAX_BBOX boxes of image 0.  The reference only
 * offers the image-file / byte-image variants (runYoloFile / runYoloList, :51-54), whose pre-processing lives in
 * its CV module outside the convolutional path. */
int runYoloNoPred(char **msg, const float *data, const int len, BBoxContainer *bboxContainer, int *detectedNum, int runGPU);
/* One 8-bit image (HWC, `channel` bytes per pixel, host memory) -> pre-processing named by preDataType (a PredDataType) on the
 * device -> forward -> index of the largest logit.  MsnhnetLib.h:44-46; the reference's own implementation needs its OpenCV
 * build (MsnhnetLib.cpp:97-...), here the facade of the build without OpenCV is followed (MsnhnetLib.cpp:540-905 over
 * src/utils/MsnhCVUtil.cpp:91-375), including what swapRGB means there: that facade exchanges the first and third channel itself
 * when swapRGB == 0 (:562, :771) and CVUtil exchanges them again by default for every variant except the letterbox, so the
 * network sees the caller's channel order when swapRGB == 0 -- except with PRE_DATA_PADDING_ZERO_FC3 and in runYoloList, where it
 * sees it when swapRGB != 0.  mean / std: three floats each, read only by PRE_DATA_TRANSFORMED_FC3.  Errors as the
 * reference's: "channel must be 1 or 3", "channel 1 must preprocess with F32_C1", "preDataType can't be none",
 * "mean or std can't be null"; 1-channel images and runGPU == 0 fail (no gray path, no CPU path in this build). */
int runClassifyList(char **msg, unsigned char *imageData, const int width, const int height, const int channel, int *bestIndex,
                    int preDataType, const int swapRGB, int runGPU, const float *mean, const float *std);
/* One 8-bit image -> letterbox (CVUtil::getPaddingZeroF32C3) -> forward -> boxes of the image in network-input pixels.
 * MsnhnetLib.h:53-54.  More than MSNHNET_MAX_BBOX boxes fail with the reference's "BBox buffer is not enough, ..." */
int runYoloList(char **msg, unsigned char *imageData, const int width, const int height, const int channel, BBoxContainer *bboxContainer,
                int *detectedNum, const int swapRGB, const int runGPU);
/* runClassifyFile / runYoloFile (MsnhnetLib.h:41-42, 51) decode image files and are not part of this library. */
int dispose(void);                                                                      /* :56 */
int withGPU(int *GPU);                                                                  /* :57 */
int withCUDNN(int *CUDNN);                                                              /* :58, always 0 */
int getCpuForwardTime(float *time);                                                     /* :59 */
int getGpuForwardTime(float *time);                                                     /* :60 */
int getInputDim(int *width, int *heigth, int *channel);                                 /* :61 */

/* ---- part 2: handle-based API (0 = success, non-zero = failure; text via msnhnet_last_error) --------------------------- */
typedef void *msnhnet_t;
const char *msnhnet_last_error(void);
int msnhnet_create(msnhnet_t *net);                       /* NetBuilder() */
int msnhnet_destroy(msnhnet_t net);
int msnhnet_set_use_fp16(int on);                         /* NetBuilder::setUseFp16, process-wide, before build */
int msnhnet_set_device_nms(int mode);                     /* hard NMS: 0 = candidates copied back, sort + NMS on the host; 2 = on the device, only kept boxes cross
                                                              PCIe; 1 (default) = chosen per batch from the previous result: on the device up to 2048 candidates per
                                                              image, and up to 6144 unless forwards are pipelined and the host keeps up with them */
int msnhnet_set_tune_cache(int on);                       /* keep the per-layer tile search result in "<weights>.f16.tune" / ".f32.tune" next to the
                                                              .msnhbin file and reuse it on the next load (same graph, same device); off by default */
int msnhnet_set_weight_cache(int on);                     /* keep the packed device-side kernels and the float16 calibration in "<weights>.f16.pack" /
                                                            * ".f32.pack" next to the weights file (NetBuilder::setWeightCache); off by default */
int msnhnet_set_use_winograd(int on);                     /* float16 builds: 3x3 stride-1 convolutions through Winograd F(2x2,3x3);
                                                             the reference keeps its own (ARM NEON, commented out) Winograd switch at
                                                             src/layers/MsnhConvolutionalLayer.cpp:1262 */
int msnhnet_set_keep_class_scores(int on);
int msnhnet_set_save_layer_output(msnhnet_t net, int on); /* NetBuilder::setSaveLayerOutput */
int msnhnet_build(msnhnet_t net, const char *msnhnet_path);      /* NetBuilder::buildNetFromMsnhNet */
int msnhnet_load(msnhnet_t net, const char *msnhbin_path);       /* NetBuilder::loadWeightsFromMsnhBin */
int msnhnet_load_from_memory(msnhnet_t net, const float *weights, size_t count);
int msnhnet_input_dims(msnhnet_t net, int *batch, int *channels, int *height, int *width);
int msnhnet_num_layers(msnhnet_t net);
/* info[0..9] = type, outH, outW, outC, outputNum, inputNum, numWeights, memReUse, batch, activation */
int msnhnet_layer_info(msnhnet_t net, int layer, long long *info, char *name, int name_cap);
long long msnhnet_layer_detail(msnhnet_t net, char *dst, long long cap);      /* returns the full length */
long long msnhnet_plan_detail(msnhnet_t net, char *dst, long long cap);
long long msnhnet_load_detail(msnhnet_t net, char *dst, long long cap);       /* wall-clock of the phases of the last load; state of the pack file */
/* The parts of the weights file this graph expects, in `.msnhbin` order (NetBuilder::loadWeightsFromMsnhBin,
 * src/net/MsnhNetBuilder.cpp:624-663, and each layer's loadAllWeigths).  parts receives up to cap triples { what, count, fan_in }:
 * what = 0 convolution / deconvolution kernel, 1 batch-norm scale, 2 batch-norm shift, 3 running mean, 4 running variance,
 * 5 bias, 6 connected weights.  Returns the number of parts (call with parts == NULL first).  Works on a built graph without weights. */
long long msnhnet_weight_layout(msnhnet_t net, long long *parts, long long cap);
double msnhnet_conv_flops(msnhnet_t net);
/* NetBuilder::runClassify / runYolo (CPU): always fail with "Gpu mode , can not run with cpu". */
int msnhnet_run_classify(msnhnet_t net, const float *img, long long n, float *out, long long cap, long long *n_out);
/* NetBuilder::runClassifyGPU: img = batch*C*H*W floats; out receives batch*outputNum floats. */
int msnhnet_run_classify_gpu(msnhnet_t net, const float *img, long long n, float *out, long long cap, long long *n_out);
/* NetBuilder::runYoloGPU: counts[b] = boxes of image b; boxes = rows of 7 floats (x y w h conf bestClsConf
 * bestClsIdx), images back to back, at most cap_boxes rows are written; *total = sum of counts. */
int msnhnet_run_yolo_gpu(msnhnet_t net, const float *img, long long n, int *counts, float *boxes, long long cap_boxes, long long *total);
/* Detectors: put the copy-back of the candidates (and the device NMS) on the forward's own stream instead of a stream of their own.
 * Off by default for a NetBuilder on its own (the copy of one batch then runs beside the next forward); the instances of a group
 * have it on (one busy stream per instance: a process has four hardware queues, and a copy stream that shares one with another
 * instance's forward waits behind that forward).  Set while nothing is in flight. */
int msnhnet_set_copy_on_forward_stream(msnhnet_t net, int on);
/* Where the hard NMS of the detection result fetched last ran: 1 on the device, 0 on the host (msnhnet_set_device_nms). */
int msnhnet_last_nms_on_device(msnhnet_t net, int *on_device);
/* Range check of a float16 plan for one input (NetBuilder::fp16Headroom): runs the network once on img and writes the factor by which
 * img could still grow before a float16 activation overflows; 0 means it already did (an input far hotter than the [0,1) image the
 * scales were calibrated on).  float32 plans report infinity. */
int msnhnet_fp16_headroom(msnhnet_t net, const float *img, long long n, float *headroom);
/* Output of top-level layer `layer` from the last run with layer dumps on (batch-major NCHW). Returns its length. */
long long msnhnet_layer_output(msnhnet_t net, int layer, float *dst, long long cap);
/* Detectors, for parity checks of the production path (no layer dumps needed).  After a fetched result:
 * msnhnet_yolo_head_logits: the input tensor of detection head `head` (heads in the order of the yoloout layer's `layers:` list) as
 *   batch-major NCHW float32, what YoloLayer::forward reads (src/layers/MsnhYoloLayer.cpp:61-142); returns its length.
 * msnhnet_yolo_candidates: the candidate rows of image `image` before sorting and suppression -- what the reference's scan keeps at
 *   src/layers/MsnhYoloOutLayer.cpp:120-170 -- 8 floats each (x y w h objectness, best class score, best class, cell number in the
 *   reference's scan order: head by head, anchor, then pixel), in no particular order; returns their number.  Available when the
 *   sort + NMS of that result ran on the host (msnhnet_set_device_nms(0)). */
long long msnhnet_yolo_head_logits(msnhnet_t net, int head, float *dst, long long cap);
long long msnhnet_yolo_candidates(msnhnet_t net, int image, float *dst, long long cap_rows);
/* Device-resident serving path: write the batch into the buffer returned by msnhnet_device_input (device memory,
 * NCHW float32) or pass another device pointer, enqueue, then sync / fetch. */
int msnhnet_device_input(msnhnet_t net, float **device_ptr);
int msnhnet_enqueue(msnhnet_t net, const float *device_input);
int msnhnet_sync(msnhnet_t net);
int msnhnet_fetch_classify(msnhnet_t net, float *out, long long cap, long long *n_out);
int msnhnet_fetch_yolo(msnhnet_t net, int *counts, float *boxes, long long cap_boxes, long long *total);
/* Upper bound of the boxes one run can return (batch * number of anchor cells); 0 for a non-detection network. */
long long msnhnet_yolo_max_boxes(msnhnet_t net);
/* Device-event timing of `reps` eager passes over the plan's launches of one kind (0 conv, 1 affine, 2 add, 3 copy,
 * 4 maxpool, 5 avgpool, 6 upsample, 7 connected, 8 input cast, 9 yolo decode, -1 all).  Outputs the total
 * milliseconds, the number of launches timed and their algorithmic FLOPs (2*MACs; 0 for non-GEMM kinds). */
int msnhnet_profile_ops(msnhnet_t net, int kind, int reps, float *ms_total, int *launches, double *flops);
/* The same with kind = 1000 + a also accepted (the convolution launches of algorithm a: 3 depthwise, 5 first layer, ...), and with
 * the bytes those launches must move at least (input + output + fused residual + weights) in *bytes. */
int msnhnet_profile_ops_bytes(msnhnet_t net, int kind, int reps, float *ms_total, int *launches, double *flops, double *bytes);
/* Per-launch timing table (text): every live launch of the plan timed on its own, `reps` repetitions each. */
long long msnhnet_profile_each_op(msnhnet_t net, int reps, char *dst, long long cap);
/* The same measurement as numbers: 8 doubles per live launch, in plan order -- kind (as msnhnet_profile_ops), convolution algorithm,
 * layer index, tile, algorithmic FLOPs, least bytes (input + output + fused residual + weights), microseconds per launch,
 * ksize * 100 + stride.  At most cap_rows rows are written; returns the number of launches. */
long long msnhnet_profile_each_op_values(msnhnet_t net, int reps, double *dst, long long cap_rows);
float msnhnet_gpu_inference_time(msnhnet_t net);          /* NetBuilder::getGpuInferenceTime, ms */
/* YoloOutLayer::nms on its own (pure host code, no GPU needed): rows of 7 floats in (x y w h conf bestClsConf
 * bestClsIdx), already in the order the layer would pass them; fast = 0 runs the reference-shaped greedy loop,
 * fast = 1 the sorted variant the library uses.  Writes at most cap rows, *n_out = number of surviving boxes. */
int msnhnet_nms(const float *rows, long long n, float nms_thresh, int fast, float *out, long long cap, long long *n_out);
/* The whole host stage of YoloOutLayer on candidate rows as msnhnet_yolo_candidates returns them (8 floats each, any order): back into
 * scan order by cell number, sorted by objectness * class score (src/layers/MsnhYoloOutLayer.cpp:175-194), then msnhnet_nms.  Pure
 * host code. */
int msnhnet_boxes_from_candidates(const float *rows8, long long n, float nms_thresh, int fast, float *out, long long cap, long long *n_out);

/* The step either side of the graph.
 * msnhnet_set_input_image_u8: letterbox one 8-bit RGB image (HWC, host memory) on the device into slot `index` of the
 *   input batch -- CVUtil::getPaddingZeroF32C3 (src/utils/MsnhCVUtil.cpp:203-261) fused with the upload; run with
 *   msnhnet_enqueue(net, NULL) afterwards.
 * msnhnet_boxes_to_image: boxes (rows of 7 floats as returned by the run / fetch calls) from network-input pixels back
 *   to the original image -- YoloOutLayer::bboxResize2Org (padded != 0) / bboxResize2OrgNoPad
 *   (src/layers/MsnhYoloOutLayer.cpp:321-379). */
int msnhnet_set_input_image_u8(msnhnet_t net, int index, const unsigned char *rgb_hwc, int width, int height, int half_init, int shuffle_rgb);
/* The same with any pre-processing variant of msnh_hip.h's msnh_preproc (plain resize + normalisation, or the letterbox). */
int msnhnet_set_input_image(msnhnet_t net, int index, const unsigned char *rgb_hwc, int width, int height, int preproc, const float *mean3,
                            const float *std3, int shuffle_rgb);
int msnhnet_boxes_to_image(float *boxes, long long count, int net_w, int net_h, int org_w, int org_h, int padded);
long long msnhnet_time_detail(msnhnet_t net, char *dst, long long cap);       /* NetBuilder::getTimeDetail */

/* Several instances of one network on one GPU, fed round-robin: the throughput arrangement for serving (no counterpart in the
 * reference, whose callers would create several NetBuilder objects and threads themselves).  Each instance is a NetBuilder with
 * its own stream, arena and graph (one packed copy of the weights serves all), driven by its own host thread with `depth` batches in flight (detectors 1 or
 * 2, classifiers 1); the device runs the forwards of different instances side by side, which fills the gaps between the launches
 * of one forward.  The switches of msnhnet_set_* apply as for msnhnet_create + build + load.
 *   msnhnet_group_prime  : one forward of the device-resident float32 NCHW batch on every instance, on the calling thread
 *                          (fills each instance's input buffer, captures its graph); call once before submitting.
 *   msnhnet_group_submit : hands the next batch to the next instance; device_input as for msnhnet_enqueue (NULL = run on what
 *                          the instance's input buffer holds), valid until the batch's result has been fetched.
 *   msnhnet_group_flush  : every instance fetches what it still holds in flight now (it otherwise keeps depth - 1 results back
 *                          until more work comes or a fetch asks for one of them).  Calls on one group come from one thread.
 *   msnhnet_group_fetch_*: the oldest outstanding result, outputs as for msnhnet_fetch_*; blocks until it is there; an error
 *                          raised inside an instance's thread is reported by the fetch of the batch it belongs to.
 *   msnhnet_group_instance: the NetBuilder of instance i (owned by the group) for the query calls: dims, plan detail, profiles. */
typedef void *msnhnet_group_t;
int msnhnet_group_create(const char *msnhnet_path, const char *msnhbin_path, int instances, int depth, msnhnet_group_t *group);
int msnhnet_group_destroy(msnhnet_group_t group);
int msnhnet_group_info(msnhnet_group_t group, int *instances, int *depth, int *is_detector);
int msnhnet_group_instance(msnhnet_group_t group, int i, msnhnet_t *net);
int msnhnet_group_prime(msnhnet_group_t group, const float *device_input);
int msnhnet_group_submit(msnhnet_group_t group, const float *device_input);
int msnhnet_group_flush(msnhnet_group_t group);
int msnhnet_group_fetch_classify(msnhnet_group_t group, float *out, long long cap, long long *n_out);
int msnhnet_group_fetch_yolo(msnhnet_group_t group, int *counts, float *boxes, long long cap_boxes, long long *total);

#ifdef __cplusplus
}
#endif
#endif
