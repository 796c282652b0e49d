/*
 * tfjs_hip.h -- C ABI of the MI355X (gfx950) native half of tfjs-backend-hip.
 *
 * One process, one GPU, one HIP stream. Every entry point returns 0 on success
 * and a non-zero status on failure; tfhip_last_error() then describes the
 * failure (the N-API shim turns it into a thrown JS Error, the convention of
 * tfjs-node/binding/utils.h:46-94). Kernel entry points only enqueue work on
 * the library's stream; tfhip_download() and tfhip_sync() are the sync points.
 *
 * Device memory is owned by the library: tfhip_alloc() hands out device
 * pointers from a size-bucketed pool and records every live block, and every
 * kernel entry point checks that each operand range lies inside a live block
 * before launching, so a wrong shape is an error return and never a GPU fault.
 *
 * All tensors are dense, row-major float32 unless stated. "Reference" citations
 * are file:line in the tensorflow/tfjs source tree and name the interface each
 * entry point stands in for.
 */
#ifndef TFJS_HIP_H_
#define TFJS_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Fused activation codes. Numbering of FusableActivation,
 * tfjs-backend-wasm/src/cc/backend.h:32-40 and
 * tfjs-backend-wasm/src/kernels/types.ts:28-36. */
enum tfhip_activation {
  TFHIP_LINEAR = 0,
  TFHIP_RELU = 1,
  TFHIP_RELU6 = 2,
  TFHIP_PRELU = 3,
  TFHIP_LEAKYRELU = 4,
  TFHIP_SIGMOID = 5,
  TFHIP_ELU = 6
};

/* ---- library lifetime ---------------------------------------------------
 * Stands in for the wasm backend's init()/dispose()
 * (tfjs-backend-wasm/src/cc/backend.h:97-120) and for the constructor of
 * TFJSBackend in the Node addon (tfjs-node/binding/tfjs_backend.cc). */
int tfhip_init(int device);
int tfhip_shutdown(void);
const char *tfhip_last_error(void);
/* name: device name; arch: gcnArchName; cus: compute units; hbm_bytes: total
 * device memory. Any out pointer may be NULL. */
int tfhip_device_info(char *name, size_t name_len, char *arch, size_t arch_len,
                      int *cus, int *clock_khz, size_t *hbm_bytes);

/* ---- buffers ------------------------------------------------------------
 * The id -> buffer bookkeeping of register_tensor()/dispose_data()
 * (tfjs-backend-wasm/src/cc/backend.h:107-115) and of createTensor /
 * deleteTensor / tensorDataSync in the Node addon
 * (tfjs-node/binding/tfjs_binding.cc:303-327). Here the handle is the device
 * pointer itself. */
int tfhip_alloc(size_t bytes, void **dptr);
int tfhip_free(void *dptr);
/* Asynchronous host->device copy of `bytes` bytes to dst (+dst_offset bytes)
 * through pinned staging; the host range may be reused on return. */
int tfhip_upload(void *dst, size_t dst_offset, const void *host, size_t bytes);
/* Waits for the stream, then copies device->host. */
int tfhip_download(void *host, const void *src, size_t src_offset, size_t bytes);
int tfhip_sync(void);
/* live: blocks handed out and not freed; live_bytes: their total size;
 * pooled_bytes: freed blocks kept for reuse. */
int tfhip_memory_info(size_t *live, size_t *live_bytes, size_t *pooled_bytes);
/* The scratch block that kernels needing device memory beyond their operands
 * share (partial sums of a matmul whose K is cut into slices). It is not a
 * tensor, so tfhip_memory_info does not count it. bytes: its present size;
 * allocations: hipMalloc calls made for it since tfhip_init; last_splits: the
 * number of K slices of the last matmul / convolution launched as a GEMM. For
 * tests and diagnosis; no counterpart in the reference. */
int tfhip_workspace_info(size_t *bytes, size_t *allocations, int *last_splits);
/* *finite = 0 when the `elems` floats at `filter` hold an Inf or a NaN, else 1.
 * The reference skips filter taps that fall outside the image
 * (tfjs-backend-cpu/src/kernels/Conv2D.ts:72-84, DepthwiseConv2dNative.ts:72-86);
 * the matrix-core kernels read a zero there and multiply it, which is the same
 * number unless the filter value is not finite. The convolution entry points
 * look for themselves and give such a filter to kernels that skip the taps; the
 * fused pair and block entry points refuse it, and this tells a caller
 * beforehand to run the separate convolutions instead. The answer is remembered
 * per filter (address, length, allocation), so asking costs one small kernel and
 * one wait for the stream the first time and a table look-up afterwards; the
 * first question about a filter cannot be asked while recording. */
int tfhip_filter_is_finite(const float *filter, int64_t elems, int *finite);
/* Lets kernels accept device memory the caller allocated elsewhere. */
int tfhip_register_external(void *dptr, size_t bytes);
int tfhip_unregister_external(void *dptr);

/* ---- timing (KernelBackend.time(), tfjs-core/src/backends/backend.ts:88-92)
 * Events are recorded on the library's stream. tfhip_event_record(slot) marks
 * slot (0..TFHIP_MAX_EVENTS-1); tfhip_event_elapsed(a, b, &ms) waits for b and
 * returns the milliseconds between the two marks. */
#define TFHIP_MAX_EVENTS 4096
int tfhip_event_record(int slot);
int tfhip_event_elapsed(int start_slot, int end_slot, float *ms);

/* ---- recorded launch sequences (no counterpart in the reference) --------------
 * A model whose shapes do not change enqueues the same kernels with the same
 * arguments at every inference. Between tfhip_capture_begin() and
 * tfhip_capture_end() the kernel entry points record their launches into a
 * HIP graph instead of running them; tfhip_graph_launch(id) then replays the
 * whole sequence with one call: no per-kernel host work, and shorter gaps
 * between dependent kernels than separate launches leave.
 *  - While recording, tfhip_alloc / tfhip_free work as usual (a block freed
 *    while recording is kept by the graph until tfhip_graph_destroy), and the
 *    entry points that wait for the stream or copy through the host
 *    (tfhip_upload, tfhip_download, tfhip_sync, the event calls) fail.
 *  - A replay reads and writes the ADDRESSES that were recorded: the caller
 *    puts new input where the recorded input was (tfhip_copy) and takes the
 *    result from where the recorded result was. Blocks that were live at
 *    tfhip_capture_end and that a recorded kernel names must still be live at
 *    every tfhip_graph_launch, which checks this and fails without launching
 *    otherwise.
 *  - tfhip_capture_end(NULL, &nodes) discards the recording.
 * nodes: kernels in the graph. */
int tfhip_capture_begin(void);
int tfhip_capture_end(int *graph_id, int *nodes);
int tfhip_graph_launch(int graph_id);
int tfhip_graph_destroy(int graph_id);

/* ---- measurement aids (no counterpart in the reference) ----------------------
 * tfhip_set_launch_repeat(n): every kernel entry point enqueues its kernel n
 *   times back to back (the kernels are idempotent), so that a pair of events
 *   around one call times n launches without n trips through the caller's
 *   language. n = 1 is normal operation.
 * tfhip_last_kernel: symbol of the kernel the last entry point chose, spelled as
 *   a profiler demangles it, e.g. "gemm_kernel<128, 128, 16, 2, 2, 0, 1, 1>".
 * tfhip_copy: a plain device-to-device copy kernel ("copy_f4": reads `bytes`,
 *   writes `bytes`; both pointers 16-byte aligned, bytes a multiple of 16): the
 *   yardstick that a kernel's bandwidth and a profiler's traffic counters are
 *   scaled by.
 * tfhip_set_tuning(name, value): overrides a kernel-selection heuristic; value < 0
 *   restores it. Knobs: "tile" (GEMM tile shape index), "splitk" (K slices),
 *   "dw_rows" (output rows per chunk of the 3x3 depthwise kernel), "dw_halo" (1: the
 *   LDS halo depthwise kernel), "no_skinny" (1: tiled GEMM also for tall products),
 *   "skinny_regs" (0: the streaming GEMM always stages B in LDS), "fuse_pw_dw"
 *   (tfhip_pointwise_depthwise_pays: 1: yes for every shape the fused kernel
 *   takes, 0: never), "pw_dw_tile" (1 / 0: the channel-sliced / the row-ring
 *   pointwise + depthwise kernel where both take a shape), "tile_slice" (32 / 48 /
 *   64 channels per workgroup of the channel-sliced kernel), "tile_chunks" (its row
 *   chunks per image), "block_rows" (output rows per workgroup of the whole-block
 *   kernel), "fuse_block" (tfhip_inverted_residual_pays: 1 always, 0 never), "k_groups" (1 / 2 / 4
 *   groups of wavefronts that share a GEMM tile and split its k loop), "pw_dw_stream"
 *   (1 / 0: the register-streaming pointwise + depthwise kernel wherever it takes the
 *   shape / never), "stream_rows" (its output rows per wavefront), "stream_blocks" (1 / 2
 *   blocks of 16 channels per wavefront), "skinny_stage" (0: the streaming GEMM never
 *   stages A in LDS). The environment variable of a knob is its name in capitals behind
 *   TFHIP_ (TFHIP_TILE, TFHIP_SPLITK, ... TFHIP_SKINNY_STAGE), read at tfhip_init(). */
int tfhip_set_launch_repeat(int n);
int tfhip_last_kernel(char *name, size_t name_len);
int tfhip_set_tuning(const char *name, int value);
int tfhip_copy(void *dst, const void *src, size_t bytes);

/* ---- _FusedMatMul / BatchMatMul ------------------------------------------
 * Replaces _FusedMatMul(a_id, a_shape, ..., out_id)
 * (tfjs-backend-wasm/src/cc/kernels/_FusedMatMul.cc:30-43) and BatchMatMul
 * (tfjs-backend-wasm/src/cc/kernels/BatchMatMul.cc); semantics of
 * tfjs-backend-cpu/src/kernels/_FusedMatMul.ts:26-62 and BatchMatMul.ts:25-133.
 *
 * a is [batch_a, M, K] (or [batch_a, K, M] if transpose_a), b is
 * [batch_b, K, N] (or [batch_b, N, K] if transpose_b); out is
 * [max(batch_a,batch_b), M, N], batch index of each operand taken modulo its
 * own batch count. bias / prelu_weights may be NULL. When present they are
 * addressed as base[bi*strides[0] + i*strides[1] + j*strides[2]] for output
 * element (bi, i, j): a stride of 0 broadcasts along that axis. */
int tfhip_fused_matmul(const float *a, const float *b, float *out,
                       int64_t batch_a, int64_t batch_b, int64_t M, int64_t N,
                       int64_t K, int transpose_a, int transpose_b,
                       const float *bias, const int64_t bias_strides[3],
                       int activation, const float *prelu_weights,
                       const int64_t prelu_strides[3], double leakyrelu_alpha);

/* tfhip_fused_matmul for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). It
 * has no counterpart in the reference. Same arguments and the same kernels; the
 * one difference is where a product whose K is cut into slices keeps its
 * partial sums: not in the library's growing workspace but in a static device
 * array of TFHIP_NOALLOC_SCRATCH_BYTES that each GPU holds until the process
 * ends. The call makes no hipMalloc / hipFree. When the slices the library
 * would choose (at most 8, and 1 whenever the tiles already fill the GPU or K
 * is short) need more than the array (slices x batch x M x N x 4 bytes), it
 * takes the largest number of slices that fits, down to one slice, which needs
 * no scratch: the result then has tfhip_fused_matmul's bits only where the two
 * slice counts agree, and is within the float32 bound otherwise. A slice count
 * the caller forced with the "splitk" knob is not reduced: if it does not fit,
 * the call fails with a message that states both sizes, and launches nothing.
 * Every call on a GPU shares that GPU's array: calls that overlap on one GPU
 * (other threads, other streams) race on it. The array belongs to the calling
 * thread for the length of the call; tfhip_fused_matmul on another thread keeps
 * the library's workspace. Nothing is cleared between calls because each call
 * writes every element it later reads. */
#define TFHIP_NOALLOC_SCRATCH_BYTES (16u << 20)
int tfhip_fused_matmul_noalloc(const float *a, const float *b, float *out,
                               int64_t batch_a, int64_t batch_b, int64_t M,
                               int64_t N, int64_t K, int transpose_a,
                               int transpose_b, const float *bias,
                               const int64_t bias_strides[3], int activation,
                               const float *prelu_weights,
                               const int64_t prelu_strides[3],
                               double leakyrelu_alpha);

/* ---- FusedConv2D -----------------------------------------------------------
 * Replaces FusedConv2D(x_id, batch_size, input_height, ..., out_id)
 * (tfjs-backend-wasm/src/cc/kernels/FusedConv2D.cc:33-54); semantics of
 * tfjs-backend-cpu/src/kernels/FusedConv2D.ts:26-95 over Conv2D.ts:23-103.
 * The caller has already run computeConv2DInfo
 * (tfjs-core/src/ops/conv_util.ts:177-236) and passes its numbers.
 *
 * x is NHWC [batch,in_h,in_w,in_c] (nchw == 0) or NCHW; filter is HWIO
 * [f_h,f_w,in_c,out_c]; y has the same data format as x. bias / prelu_weights
 * are addressed as base[n*s[0] + h*s[1] + w*s[2] + c*s[3]] for output element
 * (n, h, w, c) whatever the data format. */
int tfhip_fused_conv2d(const float *x, const float *filter, float *y,
                       int64_t batch, int64_t in_h, int64_t in_w, int64_t in_c,
                       int64_t f_h, int64_t f_w, int64_t out_c,
                       int64_t stride_h, int64_t stride_w, int64_t dilation_h,
                       int64_t dilation_w, int64_t pad_top, int64_t pad_left,
                       int64_t out_h, int64_t out_w, int nchw,
                       const float *bias, const int64_t bias_strides[4],
                       int activation, const float *prelu_weights,
                       const int64_t prelu_strides[4], double leakyrelu_alpha);

/* FusedConv2D followed by the Add of a residual connection, as one launch:
 * y = activation(conv(x, filter) + bias) + residual, every step rounded to
 * float32 like the separate kernels (so the result equals tfhip_fused_conv2d
 * followed by tfhip_add bit for bit). The pair it replaces in a graph is a
 * FusedConv2D node (tfjs-converter/src/operations/executors/
 * convolution_executor.ts:100-137) whose only consumer is an Add / AddV2 node
 * (arithmetic_executor.ts:30-37) with an operand of the output's shape, the
 * form the projection convolution and the skip connection of an inverted
 * residual block take. residual has the shape and the data format of y and
 * must not be y itself. */
int tfhip_fused_conv2d_add(const float *x, const float *filter, float *y,
                           int64_t batch, int64_t in_h, int64_t in_w, int64_t in_c,
                           int64_t f_h, int64_t f_w, int64_t out_c,
                           int64_t stride_h, int64_t stride_w, int64_t dilation_h,
                           int64_t dilation_w, int64_t pad_top, int64_t pad_left,
                           int64_t out_h, int64_t out_w, int nchw,
                           const float *bias, const int64_t bias_strides[4],
                           int activation, const float *prelu_weights,
                           const int64_t prelu_strides[4], double leakyrelu_alpha,
                           const float *residual);

/* ---- FusedDepthwiseConv2D ----------------------------------------------------
 * Replaces FusedDepthwiseConv2D(...)
 * (tfjs-backend-wasm/src/cc/kernels/FusedDepthwiseConv2D.cc); semantics of
 * tfjs-backend-cpu/src/kernels/FusedDepthwiseConv2D.ts:25-61 over
 * DepthwiseConv2dNative.ts:23-102. NHWC only; filter is
 * [f_h,f_w,in_c,ch_mul]; y is [batch,out_h,out_w,in_c*ch_mul]. */
int tfhip_fused_depthwise_conv2d(
    const float *x, const float *filter, float *y, int64_t batch, int64_t in_h,
    int64_t in_w, int64_t in_c, int64_t f_h, int64_t f_w, int64_t ch_mul,
    int64_t stride_h, int64_t stride_w, int64_t dilation_h, int64_t dilation_w,
    int64_t pad_top, int64_t pad_left, int64_t out_h, int64_t out_w,
    const float *bias, const int64_t bias_strides[4], int activation,
    const float *prelu_weights, const int64_t prelu_strides[4],
    double leakyrelu_alpha);

/* ---- pointwise + depthwise convolution in one launch ---------------------------
 * y = dw_act(depthwise3x3(pw_act(conv1x1(x, pw_filter) + pw_bias), dw_filter) + dw_bias):
 * the expansion and the depthwise stage of an inverted-residual block without the
 * expanded tensor ever reaching memory. In a graph this is a FusedConv2D node with
 * a 1x1 filter, stride 1 (convolution_executor.ts:100-137) whose only consumer is a
 * FusedDepthwiseConv2dNative node with a 3x3 filter, channel multiplier 1, dilation
 * 1 (convolution_executor.ts:139-173). Every intermediate value is rounded as the
 * two separate kernels round it (the result equals tfhip_fused_conv2d followed by
 * tfhip_fused_depthwise_conv2d). NHWC; x is [batch,in_h,in_w,in_c], pw_filter
 * [in_c,mid_c], dw_filter [3,3,mid_c], biases [mid_c] or NULL, y
 * [batch,out_h,out_w,mid_c]; stride, pad_top, pad_left, out_h, out_w are those of
 * the depthwise stage; both activations relu or both relu6.
 * The fused kernel takes in_c 8 / 16 / 24 / 32, mid_c a multiple of 16 up to
 * 256, stride 1 or 2; for any other shape or activation pair
 * tfhip_fused_pointwise_depthwise fails and the caller runs the two
 * convolutions. tfhip_pointwise_depthwise_pays returns 1 when the kernel takes
 * the shape AND is expected to be faster than the two (an expanded tensor large
 * enough that writing and re-reading it is what the pair costs): what a graph
 * executor asks before it fuses the two nodes. */
int tfhip_fused_pointwise_depthwise(const float *x, const float *pw_filter,
                                    const float *pw_bias, int pw_activation,
                                    const float *dw_filter, const float *dw_bias,
                                    int dw_activation, float *y, int64_t batch,
                                    int64_t in_h, int64_t in_w, int64_t in_c,
                                    int64_t mid_c, int64_t stride, int64_t pad_top,
                                    int64_t pad_left, int64_t out_h, int64_t out_w);
int tfhip_pointwise_depthwise_pays(int64_t batch, int64_t in_c, int64_t mid_c,
                                        int64_t stride, int64_t out_h, int64_t out_w);

/* The same with a convolution over few input channels as the first stage (a network's
 * stem followed by the first block's depthwise stage): x [batch,in_h,in_w,in_c] with
 * in_c <= 4, filter [f_h,f_w,in_c,mid_c] of at most 36 taps (f_h * f_w * in_c), its
 * stride and padding, the intermediate tensor [batch,mid_h,mid_w,mid_c], then the
 * depthwise 3x3 stage as above. The nodes it stands for are a FusedConv2D and the
 * FusedDepthwiseConv2dNative that is its only reader; the result equals
 * tfhip_fused_conv2d followed by tfhip_fused_depthwise_conv2d bit for bit.
 * tfhip_conv2d_depthwise_pays: as tfhip_pointwise_depthwise_pays. */
int tfhip_fused_conv2d_depthwise(const float *x, const float *filter, const float *bias,
                                 int activation, const float *dw_filter,
                                 const float *dw_bias, int dw_activation, float *y,
                                 int64_t batch, int64_t in_h, int64_t in_w, int64_t in_c,
                                 int64_t f_h, int64_t f_w, int64_t mid_c, int64_t stride,
                                 int64_t pad_top, int64_t pad_left, int64_t mid_h,
                                 int64_t mid_w, int64_t dw_stride, int64_t dw_pad_top,
                                 int64_t dw_pad_left, int64_t out_h, int64_t out_w);
int tfhip_conv2d_depthwise_pays(int64_t batch, int64_t in_c, int64_t f_h, int64_t f_w,
                                int64_t mid_c, int64_t mid_h, int64_t mid_w,
                                int64_t dw_stride, int64_t out_h, int64_t out_w);

/* ---- a whole inverted-residual block in one launch -------------------------------
 * y = conv1x1(dw_act(depthwise3x3(pw_act(conv1x1(x, pw) + pw_bias), dw) + dw_bias), proj) + proj_bias
 *     [+ residual]:
 * the expansion, the depthwise stage and the linear projection of an inverted-residual
 * block, and the Add of its skip connection where `residual` is not NULL, without the
 * expanded tensor or the depthwise output ever reaching memory. In a graph these are a
 * FusedConv2D node with a 1x1 filter (convolution_executor.ts:100-137), the
 * FusedDepthwiseConv2dNative node that is its only reader (3x3, channel multiplier 1,
 * dilation 1; convolution_executor.ts:139-173), the 1x1 FusedConv2D with no activation
 * that is that node's only reader, and the Add / AddV2 node (arithmetic_executor.ts:30-37)
 * that reads the projection and a tensor of its shape. Every intermediate value is
 * rounded as the separate kernels round it: the result equals tfhip_fused_conv2d,
 * tfhip_fused_depthwise_conv2d and tfhip_fused_conv2d_add in turn.
 * NHWC; x [batch,in_h,in_w,in_c]; y and residual [batch,out_h,out_w,out_c]; stride,
 * pad_top, pad_left, out_h, out_w are the depthwise stage's; `activation` (relu or
 * relu6) is that of the expansion and of the depthwise stage; the projection is linear.
 * The two 1x1 filters come TRANSPOSED, k-contiguous per output channel:
 * pw_filter_t [mid_c,in_c] and proj_filter_t [out_c,mid_c] (tfhip_transpose2d of the
 * HWIO filters' [in,out] matrices: a caller does it once per model); dw_filter is
 * [3,3,mid_c]; biases may be NULL.
 * The kernel takes in_c 32 / 64 / 96 / 160, mid_c a multiple of 64, out_c a multiple
 * of 4 up to 160, stride 1 or 2, maps up to about 28 columns wide; for any other form
 * it fails and the caller runs the separate convolutions. tfhip_inverted_residual_pays
 * returns 1 when the kernel takes the shape AND is expected to be faster than them.
 *
 * tfhip_transpose2d: y[c][r] = x[r][c] for a row-major [rows, cols] matrix (the
 * Transpose kernel of tfjs-backend-cpu/src/kernels/Transpose.ts for rank 2, perm [1,0]). */
int tfhip_fused_inverted_residual(const float *x, const float *pw_filter_t,
                                  const float *pw_bias, int activation,
                                  const float *dw_filter, const float *dw_bias,
                                  const float *proj_filter_t, const float *proj_bias,
                                  const float *residual, float *y, int64_t batch,
                                  int64_t in_h, int64_t in_w, int64_t in_c,
                                  int64_t mid_c, int64_t out_c, int64_t stride,
                                  int64_t pad_top, int64_t pad_left, int64_t out_h,
                                  int64_t out_w);
int tfhip_inverted_residual_pays(int64_t batch, int64_t in_h, int64_t in_w,
                                 int64_t in_c, int64_t mid_c, int64_t out_c,
                                 int64_t stride, int64_t out_h, int64_t out_w);
int tfhip_transpose2d(const float *x, float *y, int64_t rows, int64_t cols);

/* ---- weight dequantisation on load -----------------------------------------
 * The quantization branch of decodeWeight, tfjs-core/src/io/io_utils.ts:196-251,
 * which the reference runs in JavaScript before backend.write(). `q` points at
 * the quantized bytes on the device (any byte alignment).
 *   affine (:223-227, :243-247): bits is 8 or 16 (little-endian codes);
 *     out[i] = fround(double(q[i]) * scale + min), or, when to_int32 != 0,
 *     Int32Array-store(Math.round(double(q[i]) * scale + min)).
 *   f16 (:229-231, getFloat16Decoder :720-741): exact binary16 -> binary32. */
int tfhip_dequant_affine(const void *q, int bits, int64_t n, double scale,
                         double min, void *out, int to_int32);
int tfhip_dequant_f16(const void *q, int64_t n, float *out);

/* ---- glue kernels of a MobileNetV2 graph -------------------------------------
 * tfhip_add: broadcasting Add (tfjs-backend-cpu/src/kernels/Add.ts:23-30,
 *   utils/binary_impl.ts:25-68). out has `rank` (<= 6) dims out_shape; a and b
 *   are addressed with element strides per output dim (0 = broadcast).
 * tfhip_mean_hw: Mean over axes [1,2] of an NHWC tensor
 *   (tfjs-backend-cpu/src/kernels/Mean.ts:26-56, Sum.ts:30-92):
 *   y[n,c] = fround(sum_hw double(fround(x / fround(H*W)))). */
int tfhip_add(const float *a, const int64_t *a_strides, const float *b,
              const int64_t *b_strides, float *out, const int64_t *out_shape,
              int rank);
int tfhip_mean_hw(const float *x, float *y, int64_t batch, int64_t h, int64_t w,
                  int64_t c);
/* The other element-wise and pooling kernels a converted MobileNetV2 graph holds
 * between its fused nodes (tfjs-converter's executors arithmetic_executor.ts:30-70,
 * basic_math_executor.ts:150-160, convolution_executor.ts:219-232,
 * transformation_executor.ts:28-36):
 * tfhip_binary: op 0 Add, 1 Sub (tfjs-backend-cpu/src/kernels/Sub.ts), 2 Multiply
 *   (Multiply.ts), operands addressed as in tfhip_add.
 * tfhip_unary: the stand-alone activation kernels Relu.ts, Relu6.ts, LeakyRelu.ts,
 *   Sigmoid.ts, Elu.ts (activation codes as above; prelu and linear are not unary).
 * tfhip_avg_pool: AvgPool, NHWC (AvgPool.ts:25-58 over utils/pool_utils.ts:20-87):
 *   y = fround(sum of the window's elements inside the image, in a double / their
 *   count). The caller passes what computePool2DInfo (conv_util.ts:119-140) gave.
 * tfhip_cast: Cast.ts:28-46 between float32 (dtype 0), int32 (1) and bool (2, one
 *   byte per element): to int32 as Int32Array.from (truncate, wrap modulo 2^32, NaN
 *   and infinities 0), to bool as x != 0. */
int tfhip_binary(int op, const float *a, const int64_t *a_strides, const float *b,
                 const int64_t *b_strides, float *out, const int64_t *out_shape,
                 int rank);
int tfhip_unary(int activation, const float *x, float *y, int64_t n,
                double leakyrelu_alpha);
int tfhip_avg_pool(const float *x, float *y, int64_t batch, int64_t in_h,
                   int64_t in_w, int64_t c, int64_t f_h, int64_t f_w,
                   int64_t stride_h, int64_t stride_w, int64_t pad_top,
                   int64_t pad_left, int64_t out_h, int64_t out_w);
int tfhip_cast(const void *x, int from_dtype, void *y, int to_dtype, int64_t n);

#ifdef __cplusplus
}
#endif
#endif /* TFJS_HIP_H_ */
