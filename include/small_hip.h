/*
 * libsmall_hip -- C ABI of the MI355X (gfx950) implementation of the SMaLL layer hot path.
 *
 * Every entry point is what a binding of the reference's layer functions would call: plain
 * ints, device pointers and a HIP stream; no C++ or torch types.  The C++ header
 * include/small.h re-creates the reference's `small::` templates on top of this ABI.
 *
 * Conventions
 *   - All tensor pointers are DEVICE pointers, 16-byte aligned, in the reference's packed
 *     layout with channel block SMALL_HIP_CB (= FloatBuffer::C_ob = C_ib = QUInt8Buffer::C_ob):
 *       activations  [batch][C/16][H][W][16]
 *       conv filter  [Co/16][Ci/cib][kh][kw][cib][16]   cib = 16, or Ci when Ci is 1, 2 or 3
 *       dw filter    [C/16][kh][kw][16]
 *       bias         [C] (channel order == packed order)
 *     (reference: include/small/abstract_layer.hpp:1419-1432, include/small/buffers.hpp:33-120)
 *   - `batch` independent images lie back to back; image n of a batched call is the
 *     reference's (batch-1) call on image n: bit for bit on the uint8 path, within float32
 *     rounding on the float path (the kernel variant, and with it the summation order, is chosen
 *     from the launch shape).  The reference has no batch argument.
 *   - Pads are given in the reference's public order: top, bottom, left, right.
 *   - Output height/width follow include/small/utils.hpp:159-165 applied to the padded input.
 *   - `stream` is a hipStream_t (NULL = the default stream).  Calls are asynchronous with
 *     respect to the host; results are ordered on the stream.
 *   - Return value: SMALL_HIP_OK, or an error code.  SMALL_HIP_ESTRIDE / ECHANNELS / ESCALE are
 *     returned exactly where the reference throws std::invalid_argument
 *     (include/small/interface_abstract.hpp); the C++ header turns them back into the same
 *     exceptions with the same messages.
 *   - In-place use (out == in) is allowed for the activation entry points, as in the reference.
 */
#ifndef SMALL_HIP_H
#define SMALL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SMALL_HIP_CB 16

#define SMALL_HIP_OK 0
#define SMALL_HIP_ESTRIDE 1   /* "<op> ERROR: stride unsupported."      */
#define SMALL_HIP_ECHANNELS 2 /* "<op> ERROR: in_channels unsupported." */
#define SMALL_HIP_ESCALE 3    /* "Upsample ERROR: scale factor unsupported (only 1 or 2)." */
#define SMALL_HIP_EINVAL 4    /* null / misaligned pointer, non-positive size, Co % 16 != 0 */
#define SMALL_HIP_EHIP 5      /* a HIP runtime call failed; see small_hip_last_error() */
#define SMALL_HIP_ENOMEM 6
#define SMALL_HIP_EUNSUPPORTED 7 /* valid arguments that a specialised entry point is not built for (a model too
                                    large for one compute unit's LDS, a layer shape outside the whole-model kernels):
                                    use the general path; small_hip_last_error() says which limit was hit */

#define SMALL_HIP_ACT_NONE 0
#define SMALL_HIP_ACT_RELU 1
#define SMALL_HIP_ACT_LEAKY 2

typedef void *small_hip_stream_t;

/* The quantisation fields the reference's QUInt8Buffer carries
 * (include/small/platforms/reference/QUInt8Buffer.hpp:222-230).  Arithmetic reads `zero` of
 * the input and filter buffers and `multiplier`, `lshift`, `rshift` of the output buffer
 * (include/small/q_abstract_layer.hpp:921-938). */
typedef struct small_hip_quant
{
    int32_t zero;
    int32_t multiplier;
    int32_t lshift;
    int32_t rshift;
} small_hip_quant;

/* ---- runtime ------------------------------------------------------------------------- */
const char *small_hip_version(void);
const char *small_hip_strerror(int status);
/* message of the last failure on the calling thread */
const char *small_hip_last_error(void);
int small_hip_device_count(void);
int small_hip_set_device(int device);
/* device memory for the Buffer classes (FloatBuffer.hpp:67-78 uses posix_memalign on the host) */
int small_hip_malloc(void **ptr, size_t bytes);
int small_hip_free(void *ptr);
int small_hip_host_malloc(void **ptr, size_t bytes); /* pinned host memory */
int small_hip_host_free(void *ptr);
int small_hip_memcpy_h2d(void *dst, const void *src, size_t bytes, small_hip_stream_t stream);
int small_hip_memcpy_d2h(void *dst, const void *src, size_t bytes, small_hip_stream_t stream);
int small_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, small_hip_stream_t stream);
int small_hip_memset(void *dst, int value, size_t bytes, small_hip_stream_t stream);
int small_hip_stream_synchronize(small_hip_stream_t stream);
/* Uploads that overlap the layer calls (no counterpart in the reference, whose buffers are host memory): a caller
 * that holds host buffers uploads batch i+1 while the layers of batch i run.
 *   small_hip_upload_begin  queues a copy of `bytes` from PINNED host memory (small_hip_host_malloc) to device memory
 *                           on the calling device's copy stream (one per device, created on first use), behind the
 *                           work already queued on `after` (so that it cannot overwrite a tensor an earlier pass
 *                           still reads); returns at once with an event handle in *done;
 *   small_hip_upload_wait   makes `stream` wait for that copy without blocking the host, and releases the handle;
 *   small_hip_upload_finish blocks the host until the copy has finished (before the host block is rewritten), and
 *                           releases the handle.
 * Exactly one of wait / finish per begin.  dst must not be a tensor that work queued AFTER the begin call reads or
 * writes before it has waited for the copy: use two input tensors in turn. */
typedef void *small_hip_event_t;
int small_hip_upload_begin(void *dst, const void *src, size_t bytes, small_hip_stream_t after, small_hip_event_t *done);
int small_hip_upload_wait(small_hip_event_t done, small_hip_stream_t stream);
int small_hip_upload_finish(small_hip_event_t done);
/* Library-owned device scratch (no counterpart in the reference, whose layers work in place on the host).  Two kinds
 * of entry point lease a block per (device, stream): small_hip_conv2d_u8 / small_hip_group_conv2d_u8 (the prepared
 * filter: small_hip_conv2d_u8_prepared_filter_bytes, times the group count), and the float32 convolution entry points
 * for a few long-reduction shapes (partial sums of the equal-share split: small_hip_conv2d_f32_workspace_bytes).
 * The first such call on a stream allocates (hipMalloc); a larger request later allocates a new block and KEEPS the
 * old one, so a pointer the library handed to a queued kernel or to a captured graph stays valid; nothing is freed
 * until small_hip_workspace_release().  The pool's lock is held from the lease until the call's launches are
 * enqueued, so such calls from several host threads take turns.  Callers with a latency budget or a graph to capture
 * call small_hip_workspace_reserve() with their largest size first; every other entry point allocates nothing. */
/* make the calling device's block of `stream` at least `bytes` long now */
int small_hip_workspace_reserve(size_t bytes, small_hip_stream_t stream);
/* free every scratch block of the calling device; call when no queued kernel or live graph of that device uses
 * library scratch (it waits for the device) */
int small_hip_workspace_release(void);
/* bytes of scratch the library holds on the calling device */
size_t small_hip_workspace_held(void);
/* scratch bytes a small_hip_conv2d_f32-family call of this shape leases (0 for most shapes) */
size_t small_hip_conv2d_f32_workspace_bytes(int batch, int kernel_height, int kernel_width, int stride, int t_pad,
                                            int b_pad, int l_pad, int r_pad, int output_channels, int input_channels,
                                            int input_height, int input_width);
/* One integer of SMALL_HIP_TUNE="key=value,..." (measurement switches; nothing in production needs them), or
 * default_value.  The C++ headers read their own switches (fuse_pool, fuse_conv_dw, one_launch) through it. */
int small_hip_tune_int(const char *key, int default_value);


/* ---- float32 layers -------------------------------------------------------------------- */
/* small::Conv2D<FloatBuffer>          include/small/interface.hpp:49-56,
 *                                     include/small/interface_abstract.hpp:46-221 */
int small_hip_conv2d_f32(int batch, int kernel_height, int kernel_width, int stride, int t_pad,
                         int b_pad, int l_pad, int r_pad, int output_channels, int input_channels,
                         int input_height, int input_width, const float *input,
                         const float *filter, float *output, small_hip_stream_t stream);
/* small::PartialConv2D<FloatBuffer>   interface.hpp:94-101, interface_abstract.hpp:416-587:
 * accumulates onto the existing contents of `output` */
int small_hip_partial_conv2d_f32(int batch, int kernel_height, int kernel_width, int stride,
                                 int t_pad, int b_pad, int l_pad, int r_pad, int output_channels,
                                 int input_channels, int input_height, int input_width,
                                 const float *input, const float *filter, float *output,
                                 small_hip_stream_t stream);
/* Fused Bias + PartialConv2D + activation in one pass: the three-call sequence of
 * Conv2DLayer::compute_output (include/small/Conv2DLayer.hpp:827-879), named after
 * small::Conv2D_Bias_ReLU (include/small/fused_interface_abstract.hpp:217-290).
 * bias may be NULL; act is SMALL_HIP_ACT_*; slope is used by ACT_LEAKY only. */
int small_hip_conv2d_bias_act_f32(int batch, int kernel_height, int kernel_width, int stride,
                                  int t_pad, int b_pad, int l_pad, int r_pad, int output_channels,
                                  int input_channels, int input_height, int input_width,
                                  const float *input, const float *filter, const float *bias,
                                  int act, float slope, float *output, small_hip_stream_t stream);
/* small::Conv2D_Bias_ReLU_Maxpool2D / Conv2D_ReLU_Maxpool2D / Conv2D_Maxpool2D
 * (include/small/fused_interface_abstract.hpp:354, 998, 683) in one launch:
 *     out = MaxPool2D( act( Conv2D(in, filter) + bias ) )
 * with the pooling done on the accumulators (the convolution's own output never goes to memory; no
 * intermediate buffer is needed).  Fused here for a 2x2 stride-2 pooling window without padding (EINVAL
 * otherwise: issue the two layers); the convolution may be any this library runs except first layers with a
 * window other than 3x3.  output is [batch][Co/16][Ho/2][Wo/2][16].  The result equals the two layers run one
 * after the other bit for bit (max commutes with the monotone activations; a negative LeakyReLU slope is
 * rejected). */
int small_hip_conv2d_bias_act_maxpool2d_f32(int batch, int kernel_height, int kernel_width, int stride,
                                            int t_pad, int b_pad, int l_pad, int r_pad, int pool_kernel_height,
                                            int pool_kernel_width, int pool_stride, int pool_t_pad,
                                            int pool_b_pad, int pool_l_pad, int pool_r_pad,
                                            int output_channels, int input_channels, int input_height,
                                            int input_width, const float *input, const float *filter,
                                            const float *bias, int act, float negative_slope, float *output,
                                            small_hip_stream_t stream);
/* small::Conv2D_ReLU_DepthwiseConv2D_ReLU / Conv2D_Bias_ReLU_DepthwiseConv2D_Bias_ReLU
 * (include/small/fused_interface_abstract.hpp:1840, 1513-2500) in one launch:
 *     out = act( DepthwiseConv2D( act( Conv2D(in, filter) + bias ), dw_filter ) + dw_bias )
 * Fused here (EINVAL otherwise: issue the two layers) for
 *  - a first layer: 1-3 input channels, a 3x3 convolution of stride 1 or 2, and a 3x3 stride-1 depthwise convolution
 *    with one pixel of padding on every side;
 *  - a pointwise convolution (1x1 window, stride 1, no padding) of 16, 32, 48, 64, 96 or 128 input channels and output channels in
 *    whole groups of 32, and a 3x3 depthwise convolution of stride 1 or 2 with any padding (ESTRIDE for other strides).
 * The convolution's output never goes to memory; no intermediate buffer is needed.  dw_filter is [Co/16][3][3][16],
 * either bias may be null; one activation for both layers.  output is [batch][Co/16][Hd][Wd][16] with Hd, Wd the
 * depthwise layer's output size.  The result equals the two layers run one after the other bit for bit where the
 * stand-alone convolution adds its products in one pass (always up to 112 input channels; from 128 on it may split
 * left-over tiles along the input channels: float32 rounding then). */
int small_hip_conv2d_bias_act_dwconv2d_bias_act_f32(int batch, int kernel_height, int kernel_width, int stride,
                                                    int t_pad, int b_pad, int l_pad, int r_pad, int dw_kernel_height,
                                                    int dw_kernel_width, int dw_stride, int dw_t_pad, int dw_b_pad,
                                                    int dw_l_pad, int dw_r_pad, int output_channels,
                                                    int input_channels, int input_height, int input_width,
                                                    const float *input, const float *filter, const float *bias,
                                                    const float *dw_filter, const float *dw_bias, int act,
                                                    float negative_slope, float *output, small_hip_stream_t stream);
/* Does the library run this convolution + depthwise pair as ONE launch when both are available (the rule the entry
 * point below applies; shapes only, no pointers)?  0: no (the one-launch kernels are not built for it, or the two
 * launches are faster); 1: yes, and the result equals the two launches bit for bit; 2: yes, within float32 rounding of
 * the two launches (the stand-alone convolution may add its products in another order). */
int small_hip_conv2d_dwconv2d_one_launch_f32(int batch, int kernel_height, int kernel_width, int stride, int t_pad,
                                             int b_pad, int l_pad, int r_pad, int dw_kernel_height,
                                             int dw_kernel_width, int dw_stride, int dw_t_pad, int dw_b_pad,
                                             int dw_l_pad, int dw_r_pad, int output_channels, int input_channels,
                                             int input_height, int input_width);
/* The same pairing for ANY convolution + depthwise pair, given the intermediate buffer the reference's functions take
 * (`inter_output_buf`, include/small/fused_interface_abstract.hpp:1840-1850): [batch][Co/16][Ho][Wo][16], the
 * convolution's output size.  Succeeds wherever the two layers would.  One launch where a one-launch form exists and
 * is the faster choice (the two forms above; the intermediate buffer is then not touched), the two layers through
 * `intermediate` otherwise.  input, intermediate and output must not overlap. */
int small_hip_conv2d_bias_act_dwconv2d_bias_act_via_f32(int batch, int kernel_height, int kernel_width, int stride,
                                                        int t_pad, int b_pad, int l_pad, int r_pad, int dw_kernel_height,
                                                        int dw_kernel_width, int dw_stride, int dw_t_pad, int dw_b_pad,
                                                        int dw_l_pad, int dw_r_pad, int output_channels,
                                                        int input_channels, int input_height, int input_width,
                                                        const float *input, const float *filter, const float *bias,
                                                        const float *dw_filter, const float *dw_bias, int act,
                                                        float negative_slope, float *intermediate, float *output,
                                                        small_hip_stream_t stream);
/* PartialConv2DLayer::compute_output (include/small/PartialConv2DLayer.hpp:407-463) in one pass:
 * out = act((out + conv(in, filter)) + bias), i.e. PartialConv2D + PartialBias + activation. */
int small_hip_partial_conv2d_bias_act_f32(int batch, int kernel_height, int kernel_width, int stride,
                                          int t_pad, int b_pad, int l_pad, int r_pad,
                                          int output_channels, int input_channels, int input_height,
                                          int input_width, const float *input, const float *filter,
                                          const float *bias, int act, float negative_slope,
                                          float *output, small_hip_stream_t stream);
/* small::DepthwiseConv2D<FloatBuffer>         interface.hpp:138-145, interface_abstract.hpp:994-1051 */
int small_hip_depthwise_conv2d_f32(int batch, int kernel_height, int kernel_width, int stride,
                                   int t_pad, int b_pad, int l_pad, int r_pad, int input_channels,
                                   int input_height, int input_width, const float *input,
                                   const float *filter, float *output, small_hip_stream_t stream);
/* small::PartialDepthwiseConv2D<FloatBuffer>  interface.hpp:182-190, interface_abstract.hpp:1127-1186 */
int small_hip_partial_depthwise_conv2d_f32(int batch, int kernel_height, int kernel_width,
                                           int stride, int t_pad, int b_pad, int l_pad, int r_pad,
                                           int input_channels, int input_height, int input_width,
                                           const float *input, const float *filter, float *output,
                                           small_hip_stream_t stream);
/* Fused Bias + PartialDepthwiseConv2D + activation (DepthwiseConv2DLayer::compute_output) */
int small_hip_depthwise_conv2d_bias_act_f32(int batch, int kernel_height, int kernel_width,
                                            int stride, int t_pad, int b_pad, int l_pad, int r_pad,
                                            int input_channels, int input_height, int input_width,
                                            const float *input, const float *filter,
                                            const float *bias, int act, float slope, float *output,
                                            small_hip_stream_t stream);
/* small::MaxPool2D<FloatBuffer>       interface.hpp:276-282, interface_abstract.hpp:778-834.
 * Padded positions count as 0 (abstract_layer.hpp:514-521, 718-728). */
int small_hip_maxpool2d_f32(int batch, int kernel_height, int kernel_width, int stride, int t_pad,
                            int b_pad, int l_pad, int r_pad, int input_channels, int input_height,
                            int input_width, const float *input, float *output,
                            small_hip_stream_t stream);
/* small::AveragePool2D<FloatBuffer>   interface.hpp:316-322, interface_abstract.hpp:910-978.
 * Divides by kh*kw including padded positions (abstract_layer.hpp:565-569). */
int small_hip_avgpool2d_f32(int batch, int kernel_height, int kernel_width, int stride, int t_pad,
                            int b_pad, int l_pad, int r_pad, int input_channels, int input_height,
                            int input_width, const float *input, float *output,
                            small_hip_stream_t stream);
/* small::ReLUActivation<FloatBuffer>  interface.hpp:382-386, interface_abstract.hpp:1541-1566 */
int small_hip_relu_f32(int batch, int input_channels, int input_height, int input_width,
                       const float *input, float *output, small_hip_stream_t stream);
/* small::LeakyReLUActivation<FloatBuffer>  interface_abstract.hpp:1616-1646 (the slope arrives
 * there as a 1-element buffer; here it is passed by value) */
int small_hip_leaky_relu_f32(int batch, int input_channels, int input_height, int input_width,
                             const float *input, float negative_slope, float *output,
                             small_hip_stream_t stream);
/* small::Dropout<FloatBuffer>  interface_abstract.hpp:1697-1726: at inference a multiplication by
 * filter_buf[0] (passed here by value): out = in * scale.  In place allowed. */
int small_hip_dropout_f32(int batch, int input_channels, int input_height, int input_width,
                          const float *input, float scale, float *output, small_hip_stream_t stream);
/* small::SoftMax<FloatBuffer>  interface_abstract.hpp:1778-1832: over the WHOLE tensor of an image,
 * out = exp(in) * float(1 / sum of exp(in) over all channels and pixels); no maximum is subtracted.
 * In place allowed.  No quantised version in the reference. */
int small_hip_softmax_f32(int batch, int input_channels, int input_height, int input_width,
                          const float *input, float *output, small_hip_stream_t stream);
/* small::YOLOLayer<FloatBuffer>::compute_output   YOLOLayer.hpp:150-222: decodes a detection head.
 * input: packed [padded_channels/16][H][W][16], channel a*(5+classes)+f = field f of anchor a;
 * output: flat [batch][num_anchors*H*W][5+classes] records {cx, cy, w, h, objectness, class scores}:
 *   cx = s*(sigmoid(x)+col), cy = s*(sigmoid(x)+row), w = exp(x)*anchor_w, h = exp(x)*anchor_h, rest sigmoid(x),
 *   s = image_size / H (integer division).  anchors_wh: HOST array {w0,h0,w1,h1,...}, at most 8 anchors. */
int small_hip_yolo_decode_f32(int batch, int padded_channels, int input_height, int input_width, int num_anchors,
                              const uint32_t *anchors_wh, int num_classes, int image_size, const float *input,
                              float *output, small_hip_stream_t stream);
/* small::Accum<FloatBuffer>           interface.hpp:451-455, interface_abstract.hpp:1950-1978 */
int small_hip_accum_f32(int batch, int input_channels, int input_height, int input_width,
                        const float *input, float *output, small_hip_stream_t stream);
/* small::Bias / small::PartialBias<FloatBuffer>  interface_abstract.hpp:1992-2064 */
int small_hip_bias_f32(int batch, int num_channels, int output_height, int output_width,
                       const float *bias, float *output, small_hip_stream_t stream);
int small_hip_partial_bias_f32(int batch, int num_channels, int output_height, int output_width,
                               const float *bias, float *output, small_hip_stream_t stream);
/* small::UpSample2D<FloatBuffer>      interface.hpp:352-357, interface_abstract.hpp:1845-1889 */
int small_hip_upsample2d_f32(int batch, int scale_factor, int input_channels, int input_height,
                             int input_width, const float *input, float *output,
                             small_hip_stream_t stream);

/* small::UpSample1D<FloatBuffer>      interface_abstract_1D.hpp:1614-1660: nearest neighbour x2 along the width only;
 * `rows` is the reference's batch_size argument (independent rows of a [C/16][rows][W][16] tensor). */
int small_hip_upsample1d_f32(int batch, int scale_factor, int input_channels, int rows, int input_width,
                             const float *in, float *out, small_hip_stream_t stream);
/* small::Concat<BufferT>              interface.hpp:475-481, interface_abstract.hpp:2072-2105
 * (element_size = 4 for FloatBuffer, 1 for QUInt8Buffer) */
int small_hip_concat(int batch, uint32_t input0_channels, uint32_t input1_channels,
                     uint32_t input_height, uint32_t input_width, const void *input0,
                     const void *input1, void *output, size_t element_size,
                     small_hip_stream_t stream);
/* small::GroupConv2D<FloatBuffer> / small::PartialGroupConv2D<FloatBuffer>
 *                                      interface_abstract.hpp:1265-1328, 1402-1466
 * `groups` convolutions of `channels` -> `channels`: group g reads channels [g*channels, (g+1)*channels) of
 * the packed input, writes the same channels of the packed output and uses filter block g, each block a
 * packed Conv2D filter of channels x channels (the reference's layout on its scalar platform, where every
 * block is one element; its blocked platforms interleave 16 groups per block and feed every lane the first
 * group's input, which no caller or test of the reference relies on).  `channels` must be a multiple of 16
 * (SMALL_HIP_ECHANNELS), stride 1 or 2 (SMALL_HIP_ESTRIDE).  accumulate != 0 is the Partial form (adds into
 * the output).  One launch per image and group. */
int small_hip_group_conv2d_f32(int batch, int kernel_height, int kernel_width, int stride, int groups,
                               int t_pad, int b_pad, int l_pad, int r_pad, int channels, int input_height,
                               int input_width, const float *input, const float *filter, int accumulate,
                               float *output, small_hip_stream_t stream);
/* small::GroupConv2D<QUInt8Buffer>     interface_abstract.hpp:1332-1395 */
int small_hip_group_conv2d_u8(int batch, int kernel_height, int kernel_width, int stride, int groups,
                              int t_pad, int b_pad, int l_pad, int r_pad, int channels, int input_height,
                              int input_width, const uint8_t *input, const small_hip_quant *input_q,
                              const uint8_t *filter, const small_hip_quant *filter_q, uint8_t *output,
                              const small_hip_quant *output_q, small_hip_stream_t stream);
/* Fully connected layer y = W x, i.e. Conv2D(1,1,1,0,0,0,0,No,Ni,1,1,...) on a 1x1 image, the way
 * every reference model spells it (include/small/models/MobileNetTiny.hpp:531-538).  The
 * reference's own small::Dense (interface_abstract.hpp:2113-2132) is a per-channel scale with no
 * callers; see small_hip_dense_literal_f32. */
int small_hip_dense_f32(int batch, int output_elements, int input_elements, const float *input,
                        const float *filter, float *output, small_hip_stream_t stream);
/* small::Dense<FloatBuffer> exactly as written: out[o*Ni + i] = in[o*Ni + i] * filter[o] */
int small_hip_dense_literal_f32(int output_elements, int input_elements, const float *input,
                                const float *filter, float *output, small_hip_stream_t stream);

/* ---- quantised uint8 layers ------------------------------------------------------------- */
/* small::Conv2D<QUInt8Buffer>         interface_abstract.hpp:229-404, q_abstract_layer.hpp:894-1567 */
int small_hip_conv2d_u8(int batch, int kernel_height, int kernel_width, int stride, int t_pad,
                        int b_pad, int l_pad, int r_pad, int output_channels, int input_channels,
                        int input_height, int input_width, const uint8_t *input,
                        const small_hip_quant *input_q, const uint8_t *filter,
                        const small_hip_quant *filter_q, uint8_t *output,
                        const small_hip_quant *output_q, small_hip_stream_t stream);
/* small_hip_conv2d_u8 for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as
 * small_hip_conv2d_u8; the filter pre-pass writes into a static device array of
 * SMALL_HIP_NOALLOC_MAX_PREPARED_BYTES bytes instead of an allocated block, and the call returns SMALL_HIP_EINVAL
 * when small_hip_conv2d_u8_prepared_filter_bytes(kh, kw, Co, Ci) exceeds that (input_channels of 1..3 need no
 * scratch at all).  It calls no hipMalloc / hipFree.  Every call on one GPU shares that GPU's array.  Calls on one
 * stream are ordered by the stream; calls on different streams or host threads are ordered by the library on the
 * device (the later call's pre-pass waits for the earlier call's convolution through one event per GPU; no host
 * wait), so they are safe but do not overlap.  A call recorded into a HIP graph is not ordered that way: a replay
 * that overlaps another user of the array races, so keep replays and other calls on one stream or order them
 * yourself; the first call on a GPU (symbol lookup, event creation) must come before any capture.  Nothing in the
 * array has to start at zero: the pre-pass writes every byte the convolution reads. */
#define SMALL_HIP_NOALLOC_MAX_PREPARED_BYTES (4u << 20)
int small_hip_conv2d_u8_noalloc(int batch, int kernel_height, int kernel_width, int stride, int t_pad,
                                int b_pad, int l_pad, int r_pad, int output_channels, int input_channels,
                                int input_height, int input_width, const uint8_t *input,
                                const small_hip_quant *input_q, const uint8_t *filter,
                                const small_hip_quant *filter_q, uint8_t *output,
                                const small_hip_quant *output_q, small_hip_stream_t stream);
/* The same convolution split in two for callers whose filters are constant (the reference's
 * Conv2DLayer packs its filter once at construction, include/small/Conv2DLayer.hpp:135-341):
 * _prepare_filter re-orders a packed uint8 filter (input_channels % 16 == 0) into the kernel's
 * operand order and tabulates the per-tap filter sums the zero-point correction needs; it does
 * not depend on any zero point.  `prepared` is caller-owned device memory of
 * small_hip_conv2d_u8_prepared_filter_bytes() bytes.  small_hip_conv2d_u8 does both steps in a
 * library-owned scratch buffer on every call. */
size_t small_hip_conv2d_u8_prepared_filter_bytes(int kernel_height, int kernel_width,
                                                 int output_channels, int input_channels);
int small_hip_conv2d_u8_prepare_filter(int kernel_height, int kernel_width, int output_channels,
                                       int input_channels, const uint8_t *filter, void *prepared,
                                       small_hip_stream_t stream);
int small_hip_conv2d_u8_prepared(int batch, int kernel_height, int kernel_width, int stride,
                                 int t_pad, int b_pad, int l_pad, int r_pad, int output_channels,
                                 int input_channels, int input_height, int input_width,
                                 const uint8_t *input, const small_hip_quant *input_q,
                                 const void *prepared, const small_hip_quant *filter_q,
                                 uint8_t *output, const small_hip_quant *output_q,
                                 small_hip_stream_t stream);
/* Convolution with the element-wise tail of a residual block applied in the same pass, in place on
 * the convolution's output buffer and with that buffer's quantisation parameters -- bit-identical
 * to Conv2D(in, filter, out); [Accum(accum_input, out);] [ReLUActivation(out, out);].
 * accum_input may be NULL (no Accum); relu != 0 applies the ReLU.  No counterpart in the reference
 * (its residual blocks issue the layers separately, include/small/models/Resnet8Tiny.hpp:262-296). */
int small_hip_conv2d_accum_relu_u8(int batch, int kernel_height, int kernel_width, int stride, int t_pad,
                                   int b_pad, int l_pad, int r_pad, int output_channels,
                                   int input_channels, int input_height, int input_width,
                                   const uint8_t *input, const small_hip_quant *input_q,
                                   const uint8_t *filter, const small_hip_quant *filter_q,
                                   const uint8_t *accum_input, const small_hip_quant *accum_input_q,
                                   int relu, uint8_t *output, const small_hip_quant *output_q,
                                   small_hip_stream_t stream);
int small_hip_conv2d_accum_relu_u8_prepared(int batch, int kernel_height, int kernel_width, int stride,
                                            int t_pad, int b_pad, int l_pad, int r_pad,
                                            int output_channels, int input_channels, int input_height,
                                            int input_width, const uint8_t *input,
                                            const small_hip_quant *input_q, const void *prepared,
                                            const small_hip_quant *filter_q, const uint8_t *accum_input,
                                            const small_hip_quant *accum_input_q, int relu,
                                            uint8_t *output, const small_hip_quant *output_q,
                                            small_hip_stream_t stream);
/* small::DepthwiseConv2D<QUInt8Buffer>  interface_abstract.hpp:1059-1116 */
int small_hip_depthwise_conv2d_u8(int batch, int kernel_height, int kernel_width, int stride,
                                  int t_pad, int b_pad, int l_pad, int r_pad, int input_channels,
                                  int input_height, int input_width, const uint8_t *input,
                                  const small_hip_quant *input_q, const uint8_t *filter,
                                  const small_hip_quant *filter_q, uint8_t *output,
                                  const small_hip_quant *output_q, small_hip_stream_t stream);
/* small::MaxPool2D<QUInt8Buffer>      interface_abstract.hpp:843-899 */
int small_hip_maxpool2d_u8(int batch, int kernel_height, int kernel_width, int stride, int t_pad,
                           int b_pad, int l_pad, int r_pad, int input_channels, int input_height,
                           int input_width, const uint8_t *input, const small_hip_quant *input_q,
                           uint8_t *output, const small_hip_quant *output_q,
                           small_hip_stream_t stream);
/* small::ReLUActivation<QUInt8Buffer> interface_abstract.hpp:1577-1602 */
int small_hip_relu_u8(int batch, int input_channels, int input_height, int input_width,
                      const uint8_t *input, const small_hip_quant *input_q, uint8_t *output,
                      const small_hip_quant *output_q, small_hip_stream_t stream);
/* Fully connected uint8 layer = small::Conv2D<QUInt8Buffer>(1,1,...) on a 1x1 image */
int small_hip_dense_u8(int batch, int output_elements, int input_elements, const uint8_t *input,
                       const small_hip_quant *input_q, const uint8_t *filter,
                       const small_hip_quant *filter_q, uint8_t *output,
                       const small_hip_quant *output_q, small_hip_stream_t stream);
/* No counterpart in the reference (interface_abstract.hpp:1981 "todo", :983): defined here as
 *   Accum:        out = requant_out((in + in_q.zero) + (out + out_q.zero))
 *   AveragePool:  out = requant_out(sum over valid taps of (in + in_q.zero));
 *                 the caller folds 1/(kh*kw) into out_q.multiplier / rshift */
int small_hip_accum_u8(int batch, int input_channels, int input_height, int input_width,
                       const uint8_t *input, const small_hip_quant *input_q, uint8_t *output,
                       const small_hip_quant *output_q, small_hip_stream_t stream);
int small_hip_avgpool2d_u8(int batch, int kernel_height, int kernel_width, int stride, int t_pad,
                           int b_pad, int l_pad, int r_pad, int input_channels, int input_height,
                           int input_width, const uint8_t *input, const small_hip_quant *input_q,
                           uint8_t *output, const small_hip_quant *output_q,
                           small_hip_stream_t stream);

/* small::pack_buffer / unpack_buffer (convert_tensor2dc / convert_dc2tensor)
 * include/small/buffers.hpp:138-283, on the device: a flat [dim0][dim1][dim2][dim3] tensor (NCHW
 * activations with dim0 = 1, OIHW filters) to / from the packed layout.  type is one of
 * SMALL_HIP_INPUT .. SMALL_HIP_FILTER_FC with the reference's BufferTypeEnum meaning and the same
 * adjustments (FILTER_DW: c_ib = 1; FILTER_FC: dim2 = dim3 = 1; INPUT / FILTER_CONV with
 * dim1 < c_ib: c_ib = dim1).  element_size is 4 (float) or 1 (uint8).  batch consecutive tensors are
 * converted in one launch (no counterpart in the reference: its buffers hold one image).
 * SMALL_HIP_EINVAL where the reference prints an error and returns 0 (unknown type) or would index
 * past the tensor (extents that are not multiples of their block). */
#define SMALL_HIP_INPUT 0
#define SMALL_HIP_OUTPUT 1
#define SMALL_HIP_FILTER_DW 2
#define SMALL_HIP_FILTER_CONV 3
#define SMALL_HIP_FILTER_FC 4
int small_hip_pack(int type, int batch, uint32_t dim0, uint32_t dim1, uint32_t dim2, uint32_t dim3,
                   uint32_t c_ib, uint32_t c_ob, const void *flat, void *packed, size_t element_size,
                   small_hip_stream_t stream);
int small_hip_unpack(int type, int batch, uint32_t dim0, uint32_t dim1, uint32_t dim2, uint32_t dim3,
                     uint32_t c_ib, uint32_t c_ob, const void *packed, void *flat, size_t element_size,
                     small_hip_stream_t stream);

/* ---- a whole quantised model in one launch ------------------------------------------------------
 * No counterpart as a function in the reference; it stands for what the reference's Model classes do
 * (include/small/Model.hpp, include/small/models/Resnet8Tiny.hpp:229-414: a fixed list of layers run one after
 * the other on ping-pong buffers) for models small enough that every activation tensor and every filter fit in
 * one compute unit's 160 KB of LDS (ResNet-8 on 32x32x3: 16 KB per tensor, 77 KB of filters).  One workgroup then
 * owns one image from input to output and only those two touch device memory.  Results are bit-identical to the
 * same layers issued one by one (small_hip_conv2d_accum_relu_u8, small_hip_avgpool2d_u8, small_hip_maxpool2d_u8).
 *
 * A layer is a convolution (any window up to the tensors' one-pixel ring: pads <= 1, stride 1 or 2; a fully
 * connected layer is the 1x1 convolution on a 1x1 image; 1..3 input channels only on the model input, window up to
 * 4x4) optionally followed by Accum of another tensor and / or the in-place ReLU, or a pooling layer whose window is
 * the whole image.  Tensors are named by small integers 0..7 (re-usable like ping-pong buffers);
 * SMALL_HIP_QM_INPUT is the model input (first layer only), SMALL_HIP_QM_OUTPUT the model output (last layer only).
 * small_hip_qmodel_create() copies and re-orders the filters (it allocates device memory and returns after its
 * work on `stream` has finished; the filters may be released afterwards) and returns SMALL_HIP_EINVAL with a
 * message when the model does not fit; small_hip_qmodel_forward() is one launch and allocates nothing.
 * input: batch images back to back, packed as for small_hip_conv2d_u8; output: batch x the last layer's packed
 * output. */
#define SMALL_HIP_QL_CONV 0
#define SMALL_HIP_QL_GLOBAL_AVGPOOL 1
#define SMALL_HIP_QL_GLOBAL_MAXPOOL 2
#define SMALL_HIP_QM_INPUT (-1)
#define SMALL_HIP_QM_OUTPUT (-2)
#define SMALL_HIP_QM_NONE (-3)
typedef struct small_hip_qlayer
{
    int kind;                      /* SMALL_HIP_QL_* */
    int src, dst;                  /* tensor ids */
    int accum_src;                 /* tensor added to the convolution's output (small::Accum), or SMALL_HIP_QM_NONE;
                                      may be dst itself (a residual sum accumulated in place), never src */
    int relu;                      /* small::ReLUActivation in place on the output */
    int kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad;
    int output_channels, input_channels, input_height, input_width;
    const uint8_t *filter;         /* device pointer, packed as for small_hip_conv2d_u8; NULL for pooling */
    small_hip_quant input_q, filter_q, output_q, accum_q;   /* as the buffers of the layer-by-layer calls carry them */
} small_hip_qlayer;
typedef struct small_hip_qmodel small_hip_qmodel;
int small_hip_qmodel_create(int n_layers, const small_hip_qlayer *layers, small_hip_qmodel **model,
                            small_hip_stream_t stream);
int small_hip_qmodel_forward(const small_hip_qmodel *model, int batch, const uint8_t *input, uint8_t *output,
                             small_hip_stream_t stream);
/* bytes of one image's output / of LDS the launch uses */
size_t small_hip_qmodel_output_bytes(const small_hip_qmodel *model);
size_t small_hip_qmodel_lds_bytes(const small_hip_qmodel *model);
int small_hip_qmodel_destroy(small_hip_qmodel *model);

/* ---- 1-D layers on several rows ---------------------------------------------------------------------------------
 * reference: small::Conv1D / PartialConv1D / GroupConv1D / PartialGroupConv1D (interface_abstract_1D.hpp:47, 229, 415,
 * 1255, 1320, 1388) and small::MaxPool1D / AveragePool1D (:776, 840, 906).  A 1-D tensor is [C/16][rows][width][16]:
 * `rows` (the reference's batch_size argument) independent signals; the 1 x k window moves by `stride` along the width
 * only.  (With one row, or with stride 1, the 2-D entry points on a 1 x k window compute the same thing.)
 * groups == 0: convolution output_channels <- input_channels with optional bias / activation, accumulating onto `out`
 * when accumulate != 0; groups > 0: `groups` convolutions of input_channels -> input_channels (filter: one packed
 * Conv2D filter per group; output_channels, bias and act are not used). */
int small_hip_conv1d_f32(int batch, int kernel_width, int stride, int l_pad, int r_pad, int groups,
                         int output_channels, int input_channels, int rows, int width, const float *in,
                         const float *filter, const float *bias, int act, float slope, int accumulate, float *out,
                         small_hip_stream_t stream);
int small_hip_conv1d_u8(int batch, int kernel_width, int stride, int l_pad, int r_pad, int groups, int output_channels,
                        int input_channels, int rows, int width, const uint8_t *in, const small_hip_quant *input_q,
                        const uint8_t *filter, const small_hip_quant *filter_q, uint8_t *out,
                        const small_hip_quant *output_q, small_hip_stream_t stream);
/* is_max != 0: MaxPool1D, else AveragePool1D */
int small_hip_pool1d_f32(int is_max, int batch, int kernel_width, int stride, int l_pad, int r_pad, int channels,
                         int rows, int width, const float *in, float *out, small_hip_stream_t stream);
int small_hip_pool1d_u8(int is_max, int batch, int kernel_width, int stride, int l_pad, int r_pad, int channels,
                        int rows, int width, const uint8_t *in, const small_hip_quant *input_q, uint8_t *out,
                        const small_hip_quant *output_q, small_hip_stream_t stream);

/* ---- a whole small float32 model in one launch ---------------------------------------------------------------
 * No counterpart in the reference (it runs a model as its layer calls, include/small/models/DSCNNTiny.hpp:170-262
 * being the case this is built for): one workgroup per image keeps the activation tensors in LDS and streams each
 * layer's weights through LDS a layer ahead, so a model such as the keyword-spotting DS-CNN is one kernel instead of
 * eleven launches.  Layers: a convolution (input channels a multiple of 16, or 1..3 on the model input; any window,
 * stride 1 or 2, any padding) or a depthwise convolution, each with optional bias and ReLU / LeakyReLU as
 * small_hip_conv2d_bias_act_f32 / small_hip_depthwise_conv2d_bias_act_f32 apply them, or a pooling layer whose
 * window is the whole image; a fully connected layer is the 1x1 convolution on a 1x1 image.  Tensor ids and
 * SMALL_HIP_QM_INPUT / SMALL_HIP_QM_OUTPUT as for small_hip_qlayer.  Limits: all activation tensors that are alive
 * plus the weights of two consecutive layers within 160 KB, at most 48 KB of weights per layer; a model beyond
 * them is refused with SMALL_HIP_EINVAL and a message.  small_hip_fmodel_create() copies and re-orders filters and
 * biases (it allocates device memory and returns after its work on `stream` has finished);
 * small_hip_fmodel_forward() is one launch and allocates nothing.  Results are within the float32 tolerance of the
 * layer-by-layer calls (another summation order), not bit-identical to them. */
#define SMALL_HIP_FL_CONV 0
#define SMALL_HIP_FL_DWCONV 1
#define SMALL_HIP_FL_GLOBAL_AVGPOOL 2
#define SMALL_HIP_FL_GLOBAL_MAXPOOL 3
typedef struct small_hip_flayer
{
    int kind;                      /* SMALL_HIP_FL_* */
    int src, dst;                  /* tensor ids */
    int act;                       /* SMALL_HIP_ACT_* (convolutions) */
    float slope;                   /* LeakyReLU */
    int kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad;
    int output_channels, input_channels, input_height, input_width;   /* depthwise: output_channels is ignored */
    const float *filter;           /* device pointer, packed as for the layer-by-layer call; NULL for pooling */
    const float *bias;             /* device pointer or NULL */
} small_hip_flayer;
typedef struct small_hip_fmodel small_hip_fmodel;
int small_hip_fmodel_create(int n_layers, const small_hip_flayer *layers, small_hip_fmodel **model,
                            small_hip_stream_t stream);
int small_hip_fmodel_forward(const small_hip_fmodel *model, int batch, const float *input, float *output,
                             small_hip_stream_t stream);
/* floats of one image's output / bytes of LDS the launch uses */
size_t small_hip_fmodel_output_elems(const small_hip_fmodel *model);
size_t small_hip_fmodel_lds_bytes(const small_hip_fmodel *model);
int small_hip_fmodel_destroy(small_hip_fmodel *model);

#ifdef __cplusplus
}
#endif
#endif /* SMALL_HIP_H */
