/*
 * bbhip — C ABI of the MI355X (gfx950) differentiable-LUT library.
 *
 * Every entry point replaces one device entry point of BinaryBrain's CUDA library (declared in the reference's
 * include/bbcu/bbcu.h; the file:line each one replaces is cited below).  The reference's entry points are C++
 * function templates on the LUT width N; here N is the leading `int n` argument (2..6).  Otherwise the argument
 * lists, their order and meaning are the reference's.
 *
 * Conventions (identical to the reference unless noted):
 *   - all pointers are DEVICE pointers; the caller owns every buffer;
 *   - frame buffers are node-major, frame-minor: element (node, frame) of an fp32 buffer is p[node*frame_stride + frame];
 *     of a bit-packed buffer, bit (frame & 31) of the 32-bit word p[node*frame_stride + (frame >> 5)];
 *     `frame_stride` counts elements (floats or 32-bit words) per node row;
 *   - W and dW are [node_size][2^n] row-major fp32, input_index is [node_size][n] int32;
 *   - y and dx are write-only, dW accumulates (dW += ...), running_mean/running_var are read-modify-write;
 *   - the last argument is a hipStream_t passed as void* (NULL = the default stream); launches are asynchronous;
 *   - return value: 0 on success; non-zero on a rejected argument or a HIP error (the reference prints and blocks on
 *     stdin instead, include/bbcu/bbcu_util.h:17-36) — bbhip_GetLastErrorString() describes the last failure.
 *
 * Internal scratch (transformed tables, per-slab partial sums) comes from a library-owned arena that grows with
 * hipMalloc on demand and is reused by later calls; calls that overlap on one device (different host threads or
 * streams) race on it, exactly as the reference's allocator singleton is not thread-safe (cuda/LocalHeap.cu:174).
 * A block that the arena outgrows stays allocated until bbhip_ReleaseScratch, so kernels already queued and HIP graphs
 * captured earlier keep valid addresses; the arena never grows while the call's stream is being captured (the call fails
 * with a message instead: run it once before the capture, or bbhip_ReserveScratch).
 */
#ifndef BBHIP_H_
#define BBHIP_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- device runtime shim (reference: include/bbcu/bbcu.h:49-55, cuda/Manager.cu) ---- */
int  bbhip_GetDeviceCount(void);
int  bbhip_GetDevice(void);
void bbhip_SetDevice(int device);
void bbhip_SetHostOnly(int host_only);
int  bbhip_IsHostOnly(void);
int  bbhip_IsDeviceAvailable(void);
const char *bbhip_GetLastErrorString(void);

/* ---- caching device allocator (reference: include/bbcu/bbcu.h:63-67, cuda/LocalHeap.cu:88-139) ---- */
void  *bbhip_LocalHeap_Malloc(size_t size);
void   bbhip_LocalHeap_Free(void *ptr);
size_t bbhip_LocalHeap_GetMaxAllocSize(void);
size_t bbhip_LocalHeap_GetAllocatedSize(void);
void   bbhip_LocalHeap_GarbageCollect(void);

/* ---- raw device / pinned-host memory and copies (reference: bbcu::Malloc/Free/MallocHost/FreeHost/Memcpy,
 * include/bbcu/bbcu_util.h:89-134; Malloc/Free go through the caching allocator above) ----
 * kind: 1 = host to device, 2 = device to host, 3 = device to device.  Copies and Memset are synchronous with respect
 * to the host and ordered after work queued on the default stream. */
int bbhip_Malloc(void **ptr, size_t size);
int bbhip_Free(void *ptr);
int bbhip_MallocHost(void **ptr, size_t size);
int bbhip_FreeHost(void *ptr);
int bbhip_Memcpy(void *dst, void const *src, size_t size, int kind);
int bbhip_Memset(void *dev_ptr, int value, size_t size);
int bbhip_DeviceSynchronize(void);

/* ---- scratch arena of the current device (no counterpart in the reference: its entry points take dx_tmp from the caller
 * and allocate their other temporaries through the LocalHeap singleton) ----
 * ReserveScratch grows the arena to at least `bytes` now, so that later calls (in particular captured ones) find it large
 * enough.  ReleaseScratch waits for the device and frees the arena together with every block it has outgrown: HIP graphs
 * captured before it must not be replayed afterwards.  GetScratchSize: bytes the arena holds at present. */
int    bbhip_ReserveScratch(size_t bytes);
int    bbhip_ReleaseScratch(void);
size_t bbhip_GetScratchSize(void);

/* ---- state of an environment switch as the library read it (instrumentation; no counterpart in the reference) ----
 * name "corner" (BBHIP_CORNER: lookup kernels for two-valued inputs) or "pack" (BBHIP_PACK: binarized fp32 frames are
 * packed to bits first): 1 on, 0 off, -1 unknown name.  A switch is off when its variable is 0 (or 2), on for any other
 * number, and takes its default (on) when unset. */
int bbhip_GetSwitch(char const *name);

/* ---- how dx is accumulated over the fan-out of an input node (no counterpart in the reference) ----
 * 0 (default): deterministic, no scratch — one wavefront per (input node, frame chunk) walks reverse_index in the
 *              reference's order (cuda/Common.cuh:174-202, include/bb/FixedSizeConnectionTable.h:198-214) and
 *              re-evaluates each consumer's dy/dx from that consumer's other inputs; needs reverse_index, ignores dx_tmp.
 * 1          : fp32 atomic adds into a zero-filled dx; dx_tmp and reverse_index may be NULL; summation order is
 *              not reproducible between runs.
 * 2          : the reference's scheme — per-connection gradients go to dx_tmp ([output_node_size*n][tmp_frame_stride],
 *              tmp_frame_size frames per pass) and are summed through reverse_index; deterministic. */
void bbhip_SetDxMode(int mode);
int  bbhip_GetDxMode(void);

/* ---- number of input node rows for the next forward call (no counterpart in the reference) ----
 * The forward entry points keep the reference's signatures, which do not say how many rows the input buffer has
 * (input_index names them).  A caller that knows may say so right before a forward call of the same thread: in binary
 * mode on fp32 frames the library then packs the binarized input to bits once (it has to know how many rows to pack)
 * and runs the packed-bit kernels, as the backward entry points — which are told input_node_size — always do.
 * The hint holds for one forward call and is cleared by it; 0 clears it.  The rows [0, input_node_size) of the input
 * buffer must exist and input_index must name no row beyond them (only the named rows are read without the hint, all
 * of them with it): the value is trusted like the sizes of any entry point.  Results do not depend on the hint. */
void bbhip_HintInputNodeSize(int input_node_size);

/* ---- a caller-owned place for the packed copy of a binarized fp32 input (no counterpart in the reference) ----
 * In binary mode on fp32 frames a LUT layer reads bits: the forward and the backward entry each pack the binarized input once
 * (bit = x > 0.5) into the library's scratch, because the entry points share no state.  A caller that keeps the layer's input
 * between the two calls anyway (the model classes do) can keep the packed copy as well and save the backward pass its packing:
 *   - right before the forward call, with holds_input = 0: dev_bits, `rows` rows (the input's node count: this also serves as
 *     bbhip_HintInputNodeSize) of row_words 32-bit words each, receives the packed copy instead of the library's scratch;
 *   - right before the backward call on the same input, with holds_input = 1: the buffer still holds that copy (the caller's
 *     promise: x has not changed since), and the call reads it instead of packing x again.  A forward call takes holds_input = 1 the
 *     same way (the buffer was filled as the packed output of the layer before, bbhip_HintPackedOutput, or by an earlier call).
 * row_words must be a multiple of 8 and at least ceil(frame_size / 32) (bbhip_PackedRowWords(frame_size) gives the pitch the
 * library itself would use), dev_bits 32-byte aligned; a buffer that does not fit the call is ignored (the library packs into its
 * scratch as always).  Like the other hint it holds for the next LUT call of the same thread and is cleared by any entry.
 * Results do not depend on it. */
int  bbhip_PackedRowWords(int frame_size);
void bbhip_HintPackedInput(int *dev_bits, int rows, int row_words, int holds_input);

/* ---- the binarized output of a forward call as packed bits as well (no counterpart in the reference) ----
 * A layer in binary mode that follows another reads bits, and what it would pack is the output that the layer before has just
 * binarized.  Given right before a forward call whose output is binarized fp32 (the fp32 entries in binary mode), the call writes its
 * output to dev_y_buf as always AND as packed bits to dev_bits (`rows` = node_size rows of row_words words, row_words a multiple of 8
 * and at least ceil(frame_size / 32), 32-byte aligned; bit f & 31 of word f >> 5 = y > 0.5, words behind the last frame 0): the
 * wavefront that binarizes 64 frames stores their ballot, no extra launch.  The caller then hands that buffer to the next layer's
 * forward call as bbhip_HintPackedInput(dev_bits, rows, row_words, 1) — "this already holds the packed copy of the input" — and that
 * call packs nothing; its backward call takes it the same way.  holds_input = 1 is the caller's promise that the fp32 buffer has not
 * been written since.  A buffer that does not fit the call is ignored and not written.  Thread-local and spent by the next entry
 * called on the thread, like the other hints; the fp32 output is the same bits with and without it. */
void bbhip_HintPackedOutput(int *dev_bits, int rows, int row_words);

/* ---- table gradient written instead of accumulated (no counterpart in the reference) ----
 * The backward entries add into dev_dW, as the reference's do (dW accumulates until the optimizer or ZeroGrad clears it).  A caller
 * whose dW holds nothing worth keeping (it would zero it first) says so right before the backward call with overwrite = 1, and the
 * call writes dW = (this call's gradient) in the launch that already folds the partial sums: the caller's fill launch falls away.
 * Same bits as zero-fill followed by the plain call.  Thread-local, spent by the next entry called on the thread. */
void bbhip_HintTableGradientOverwrite(int overwrite);

/* No counterpart in the reference.  A caller-owned device buffer (256-byte aligned, bbhip_PreparedTablesBytes(n, node_size) bytes) for the
 * tables that a LUT call derives from W before its kernels run (centred coefficients, corner values).  Given right before a forward call
 * (holds_tables = 0), the call writes them there instead of into the library's scratch memory; given right before the backward call of
 * the same step with holds_tables = 1, that call takes them from there and skips its own preparation launch.  holds_tables = 1 is the
 * caller's promise that W, the LUT width, the node count, lut_binarize, unbinarize_bias (the corner values depend on it) and the kind of
 * input (two-valued or not) are those of the call
 * that filled the buffer; a buffer that is too small or not aligned is ignored and not written.  Thread-local, spent by the next entry
 * point called on the thread, like the other hints; results are the same bits with and without it. */
void   bbhip_HintPreparedTables(float *dev_tables, size_t bytes, int holds_tables);
size_t bbhip_PreparedTablesBytes(int n, int node_size);

/* ---- kernel timer (instrumentation; no counterpart in the reference) ----
 * While enabled, every call brackets its dominant kernel (which: 0 = LUT forward kernel, 1 = LUT backward kernel,
 * 2 = BinaryLut6 kernel, 3 = input-centric dx kernel, 4 = the kernels of any other entry: vector operations, Adam, Im2Col,
 * Col2Im, pooling, AverageLut, loss, accuracy) with HIP events on the launch stream.  Read waits for the recorded launches of one kind,
 * returns their summed duration and count, and forgets them. */
void bbhip_KernelTimer_Enable(int enable);
int  bbhip_KernelTimer_Read(int which, float *total_ms, int *launches);

/* ---- elementwise helpers ---- */
/* bbcu_fp32_Vector_set, include/bbcu/bbcu.h:89-94 */
int bbhip_fp32_Vector_set(float *dev_dst, float a, int size, void *stream);
/* bbcu_fp32_Vector_clamp, include/bbcu/bbcu.h:191-198 (W is clamped to [0,1] before every StochasticLut forward,
 * include/bb/StochasticLutN.h:451) */
int bbhip_fp32_Vector_clamp(float *dev_dst, float const *dev_src, float lo, float hi, int size, void *stream);
/* bbcu_fp32_Vector_add_ex, include/bbcu/bbcu.h:96-107:  dst = a * src0 + b * src1 + c.
 * These elementwise operations evaluate the reference's C++ expressions (include/bb/TensorOperator.h:41-238) in fp32
 * operation by operation (no fused multiply-add); dst may alias a source. */
int bbhip_fp32_Vector_add_ex(float *dev_dst, float const *dev_src0, float const *dev_src1, float a, float b, float c,
                             int size, void *stream);
/* bbcu_fp32_Vector_mul_ex, include/bbcu/bbcu.h:109-119:  dst = a * src0 * src1 + b */
int bbhip_fp32_Vector_mul_ex(float *dev_dst, float const *dev_src0, float const *dev_src1, float a, float b,
                             int size, void *stream);
/* bbcu_fp32_Vector_div_ex, include/bbcu/bbcu.h:121-132:  dst = (a * src0 + b) / (c * src1 + d) */
int bbhip_fp32_Vector_div_ex(float *dev_dst, float const *dev_src0, float const *dev_src1, float a, float b, float c,
                             float d, int size, void *stream);
/* bbcu_fp32_Vector_sqrt, include/bbcu/bbcu.h:134-140 (the reference launches one block of 1024 threads and so only
 * handles the first 1024 elements, cuda/Vector.cu:233; here every element is processed, as on its CPU path) */
int bbhip_fp32_Vector_sqrt(float *dev_dst, float const *dev_src, int size, void *stream);
/* bbcu_fp32_Vector_exp, include/bbcu/bbcu.h:143-149 (same remark) */
int bbhip_fp32_Vector_exp(float *dev_dst, float const *dev_src, int size, void *stream);
/* bbcu_fp32_Vector_min / min_v / max / max_v, include/bbcu/bbcu.h:152-189; std::min / std::max semantics of the CPU
 * path (include/bb/TensorOperator.h:170-222): a NaN in the second operand is dropped, in the first it propagates */
int bbhip_fp32_Vector_min(float *dev_dst, float const *dev_src0, float const *dev_src1, int size, void *stream);
int bbhip_fp32_Vector_min_v(float *dev_dst, float const *dev_src, float a, int size, void *stream);
int bbhip_fp32_Vector_max(float *dev_dst, float const *dev_src0, float const *dev_src1, int size, void *stream);
int bbhip_fp32_Vector_max_v(float *dev_dst, float const *dev_src, float a, int size, void *stream);

/* ---- Adam ---- */
/* bbcu_fp32_OptimizerAdam, include/bbcu/bbcu.h:1560-1572 (cuda/OptimizerAdam.cu:12-84).  One update of `size` tensors:
 * the four pointer tables and the element-count table are DEVICE arrays of `size` entries.  lr_t is the
 * bias-corrected rate the caller computes (include/bb/OptimizerAdam.h:171).  Per element, each step rounded to fp32:
 *     m += (1-beta1)*(g - m);   v += (1-beta2)*(g*g - v);   p -= (lr_t*m) / (sqrt(v) + 1e-7)
 * (the reference's host path, include/bb/OptimizerAdam.h:173-176; its CUDA kernel adds the 1e-7 in double). */
int bbhip_fp32_OptimizerAdam(int size, int const *dev_size_table, float *const *dev_params_buf_table,
                             float *const *dev_grads_buf_table, float *const *dev_m_buf_table,
                             float *const *dev_v_buf_table, float lr_t, float beta1, float beta2, void *stream);
/* No single counterpart in the reference: Optimizer::Update() is Step() followed by ZeroGrad() (include/bb/Optimizer.h:31-35,
 * include/bb/OptimizerAdam.h:132-139), i.e. bbcu_fp32_OptimizerAdam and then one fill per gradient tensor.  This entry does
 * both: the same update as bbhip_fp32_OptimizerAdam, and every gradient element is set to 0 once it has been used. */
int bbhip_fp32_OptimizerAdam_Update(int size, int const *dev_size_table, float *const *dev_params_buf_table,
                                    float *const *dev_grads_buf_table, float *const *dev_m_buf_table,
                                    float *const *dev_v_buf_table, float lr_t, float beta1, float beta2, void *stream);

/* bbcu_ConvBitToReal<float>, include/bbcu/bbcu.h:246-258 */
int bbhip_fp32_ConvBitToReal(int const *dev_x_buf, float *dev_y_buf, float value0, float value1,
                             int node_size, int frame_size, int x_frame_stride, int y_frame_stride, void *stream);

/* ---- convolution plumbing: Im2Col, Col2Im, StochasticMaxPooling2x2 ----
 * A convolution is Im2Col -> LUT layers -> Col2Im.  Buffers are node-major / frame-minor as everywhere; nodes are
 * (c, y, x) row-major pixels or (c, fy, fx) filter taps; Im2Col's output frame is (input frame, oy, ox) row-major.
 * Results follow the reference's host paths (include/bb/ConvolutionIm2Col.h:370-452, ConvolutionCol2Im.h:203-293,
 * StochasticMaxPooling2x2.h:190-306) bit for bit. */
/* bbcu_fp32_Im2Col_Forward, include/bbcu/bbcu.h:1076-1097.  x_stride / y_stride are the window steps, x_offset / y_offset
 * the padding ((filter-1)/2 for "same", 0 for "valid"); border_mode 0 constant (border_value), 1 reflect, 2 reflect_101,
 * 3 replicate, 4 wrap (include/bb/DataType.h BB_BORDER_*). */
int bbhip_fp32_Im2Col_Forward(float const *dev_x_buf, float *dev_y_buf, int x_stride, int y_stride, int x_offset, int y_offset,
                              int input_frame_size, int input_frame_stride, int input_w_size, int input_h_size, int input_c_size,
                              int output_w_size, int output_h_size, int output_frame_stride, int filter_w_size, int filter_h_size,
                              int border_mode, float border_value, void *stream);
/* bbcu_bit_Im2Col_Forward, include/bbcu/bbcu.h:1099-1119 (packed bits; strides in 32-bit words; constant border = 0) */
int bbhip_bit_Im2Col_Forward(int const *dev_x_buf, int *dev_y_buf, int x_stride, int y_stride, int x_offset, int y_offset,
                             int input_frame_size, int input_frame_stride, int input_w_size, int input_h_size, int input_c_size,
                             int output_w_size, int output_h_size, int output_frame_stride, int filter_w_size, int filter_h_size,
                             int border_mode, void *stream);
/* bbcu_fp32_Im2Col_Backward, include/bbcu/bbcu.h:1122-1141: dx is overwritten; only taps inside the image carry gradient */
int bbhip_fp32_Im2Col_Backward(float const *dev_dy_buf, float *dev_dx_buf, int x_stride, int y_stride, int x_offset, int y_offset,
                               int input_frame_size, int input_frame_stride, int input_w_size, int input_h_size, int input_c_size,
                               int output_w_size, int output_h_size, int output_frame_stride, int filter_w_size, int filter_h_size,
                               void *stream);
/* bbcu_fp32_Col2Im_Forward, include/bbcu/bbcu.h:1148-1159: y[(c, xy)][f] = x[c][f*h*w + xy]; input_* describe the
 * [c][frames*h*w] buffer, output_* the [c*h*w][frames] buffer (also in Backward, where the first is dx) */
int bbhip_fp32_Col2Im_Forward(float const *dev_x_buf, float *dev_y_buf, int w_size, int h_size, int c_size, int input_frame_stride,
                              int output_frame_size, int output_frame_stride, void *stream);
/* bbcu_bit_Col2Im_Forward, include/bbcu/bbcu.h:1161-1172 */
int bbhip_bit_Col2Im_Forward(int const *dev_x_buf, int *dev_y_buf, int w_size, int h_size, int c_size, int input_frame_stride,
                             int output_frame_size, int output_frame_stride, void *stream);
/* bbcu_fp32_Col2Im_Backward, include/bbcu/bbcu.h:1175-1186 */
int bbhip_fp32_Col2Im_Backward(float const *dev_dy_buf, float *dev_dx_buf, int w_size, int h_size, int c_size, int input_frame_stride,
                               int output_frame_size, int output_frame_stride, void *stream);
/* bbcu_fp32_StochasticMaxPooling2x2_Forward, include/bbcu/bbcu.h:768-780: y = 1 - prod over the 2 x 2 window of (1 - x);
 * output sizes are ceil(input / 2), window taps outside the image are skipped */
int bbhip_fp32_StochasticMaxPooling2x2_Forward(float const *dev_x_buf, float *dev_y_buf, int input_w_size, int input_h_size,
                                               int output_w_size, int output_h_size, int c_size, int frame_size, int frame_stride,
                                               void *stream);
/* bbcu_fp32_StochasticMaxPooling2x2_Backward, include/bbcu/bbcu.h:783-796 */
int bbhip_fp32_StochasticMaxPooling2x2_Backward(float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, int input_w_size,
                                                int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size,
                                                int frame_stride, void *stream);

/* ---- AverageLut, softmax cross entropy, categorical accuracy (the tail of a LUT classifier) ---- */
/* bbcu_AverageLut_Forward<float>, include/bbcu/bbcu.h:321-334.  s = sum over the n inputs dev_input_index[node*n + i] of x (each
 * replaced by +1 / -1 on x > 0 when binarize_input); with binarize_output y = +1 / -1 on s > 0, else y = s * (1 / n) with the fp32
 * reciprocal of n, as the CUDA kernel of that name writes it (cuda/AverageLut.cu:46-54, 93) — the mean, whose gradient dy / n is
 * what both backward paths of the reference return. */
int bbhip_fp32_AverageLut_Forward(float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index, int n, int node_size, int frame_size,
                                  int frame_stride, int binarize_input, int binarize_output, void *stream);
/* The same with the convention of the reference's HOST loop, which disagrees with its CUDA kernel: without binarize_output the SUM s is
 * written (include/bb/AverageLut.h:331-343).  No bbcu counterpart; for callers that reproduce networks trained on the reference's
 * host path (bb::AverageLut takes it after the command "host_sum true").  Binarized outputs are the same in both. */
int bbhip_fp32_AverageLut_ForwardSum(float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index, int n, int node_size, int frame_size,
                                     int frame_stride, int binarize_input, int binarize_output, void *stream);
/* bbcu_bit_AverageLut_Forward, include/bbcu/bbcu.h:336-346: packed bits, y = strict majority of the n inputs (a tie of an even
 * n gives 0); frame_stride in 32-bit words */
int bbhip_bit_AverageLut_Forward(int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, int n, int node_size, int frame_size,
                                 int frame_stride, void *stream);
/* bbcu_AverageLut_Backward<float>, include/bbcu/bbcu.h:348-361: dx[input] = sum of dy[node] / n over the table entries that name the
 * input, in table order (the order of the host loop, include/bb/AverageLut.h:395-404); inputs that no node names, and
 * the padding of every row, are written as 0.  Deterministic: the reverse wiring is built on the device in library scratch. */
int bbhip_fp32_AverageLut_Backward(float const *dev_dy_buf, float *dev_dx_buf, int const *dev_input_index, int n, int input_node_size,
                                   int output_node_size, int frame_size, int frame_stride, void *stream);
/* The tail of a LUT classifier in ONE launch (no counterpart in the reference, which calls the four parts one by one; for training
 * loops at small batches, where each of those launches costs its latency rather than its work):
 *   y  = bbhip_fp32_AverageLut_Forward(x) without binarize_output (output_sum = 1: bbhip_fp32_AverageLut_ForwardSum), ch_size nodes of n inputs;
 *   dy, loss = bbhip_fp32_LossSoftmaxCrossEntropy(y, t) with pix_size 1;   accuracy, category = bbhip_fp32_MetricsCategoricalAccuracy(y, t);
 *   dx = bbhip_fp32_AverageLut_Backward(dy)
 * with the same bits in every output as those calls give.  dev_y_buf, dev_dy_buf ([ch_size][frame_stride]), dev_accuracy_buf and
 * dev_category_buf ([frame_size]) may be NULL where the caller does not want them; dev_dx_buf [input_node_size][frame_stride] and
 * dev_loss_buf [frame_size] are always written.  Limits: ch_size <= 16 and 256 * (input_node_size + 32) + 4 * ch_size * n <= 65536
 * (the per-input sums of 64 frames and the table are kept in LDS: 192 input nodes with 2048 table entries, 216 with 512); larger tails
 * are rejected — call the parts. */
int bbhip_fp32_ClassifierTail_ForwardBackward(float const *dev_x_buf, float *dev_y_buf, float *dev_dx_buf, int const *dev_input_index,
                                              float const *dev_t_buf, float *dev_dy_buf, double *dev_loss_buf, int *dev_accuracy_buf,
                                              int *dev_category_buf, float t_sum, int n, int input_node_size, int ch_size, int frame_size,
                                              int frame_stride, int binarize_input, int output_sum, void *stream);
/* ---- MaxLut ----
 * The largest of n wired inputs, as the reference's host loop computes it (include/bb/MaxLut.h:293-318, 394-424): the running
 * maximum starts at -1 and is replaced by strictly larger values, so the output is never below -1 (the reference's device kernel
 * starts from the lowest float, cuda/MaxLut.cu:29) and the gradient goes to the first largest input.  binarize_input (read by the
 * device kernel only, cuda/MaxLut.cu:33-36): inputs count as +1 where positive, else -1.  Bit-exact; the backward passes add in
 * table order and give the same bits on every run. */
/* bbcu_MaxLut_Forward<float>, include/bbcu/bbcu.h:368-381 */
int bbhip_fp32_MaxLut_Forward(float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index, int n, int node_size, int frame_size,
                              int frame_stride, int binarize_input, int binarize_output, void *stream);
/* bbcu_bit_MaxLut_Forward, include/bbcu/bbcu.h:383-393: the OR of the inputs */
int bbhip_bit_MaxLut_Forward(int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, int n, int node_size, int frame_size,
                             int frame_stride, void *stream);
/* bbcu_MaxLut_Backward<float>, include/bbcu/bbcu.h:395-410; dx is overwritten (padding columns included, with zeros) */
int bbhip_fp32_MaxLut_Backward(float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, int const *dev_input_index, int n,
                               int input_node_size, int output_node_size, int frame_size, int frame_stride, int binarize_input, void *stream);
/* bbcu_bit_MaxLut_Backward<float>, include/bbcu/bbcu.h:413-427: packed x (rows of x_frame_stride words), fp32 dy and dx */
int bbhip_bit_fp32_MaxLut_Backward(int const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, int const *dev_input_index, int n,
                                   int input_node_size, int output_node_size, int frame_size, int x_frame_stride, int dy_frame_stride,
                                   void *stream);

/* ---- Reduce ----
 * Output node o is the mean of the input nodes o, O + o, 2 O + o, ...; backward hands dy / mux to each of them
 * (include/bb/Reduce.h:172-190, 229-247).  These three have no counterpart in include/bbcu/bbcu.h: the reference runs this layer
 * on the host (its device calls are compiled out, Reduce.h:150-170, 207-227), which costs a device-resident pipeline a round trip
 * through host memory.  Bit-exact with the host loops. */
int bbhip_fp32_Reduce_Forward(float const *dev_x_buf, float *dev_y_buf, int input_node_size, int output_node_size, int frame_size,
                              int frame_stride, void *stream);
/* packed input (rows of x_frame_stride words) read as +1 / -1 */
int bbhip_bit_fp32_Reduce_Forward(int const *dev_x_buf, float *dev_y_buf, int input_node_size, int output_node_size, int frame_size,
                                  int x_frame_stride, int y_frame_stride, void *stream);
int bbhip_fp32_Reduce_Backward(float const *dev_dy_buf, float *dev_dx_buf, int input_node_size, int output_node_size, int frame_size,
                               int frame_stride, void *stream);

/* ---- RealToBinary, BinaryToReal ----
 * The converters at either end of a binary network (include/bb/BinaryModulation.h:44-46).  Results are the bits of the reference's
 * host loops evaluated in fp32 without fused multiply-adds. */
/* bbcu_RealToBinary_Forward<float>, include/bbcu/bbcu.h:1337-1352 (host loop include/bb/RealToBinary.h:300-344, no value generator):
 * input node (depth c, point p) and frame g give output node (depth c * depth_modulation_size + d, point p), frame
 * g * frame_modulation_size + f the value  clamp01((((x - lo) / (hi - lo)) - d / dm) * dm - f / fm) * fm), and +1 / -1 by > 0.5 when
 * `binarize`.  A NaN input gives 1. */
int bbhip_fp32_RealToBinary_Forward(float const *dev_x_buf, float *dev_y_buf, unsigned depth_modulation_size, unsigned frame_modulation_size,
                                    float input_range_lo, float input_range_hi, unsigned point_size, unsigned x_depth_size,
                                    unsigned x_frame_size, unsigned x_frame_stride, unsigned y_frame_stride, int binarize, void *stream);
/* bbcu_bit_RealToBinary_Forward<float>, include/bbcu/bbcu.h:1355-1370, packed output (rows of y_frame_stride words; bits past the
 * last frame of a row's last word are written as 0).  `binarize` is not in the reference's signature: its device kernel always takes
 * the bit as value > 0.5 (pass 1 for that), its host loop takes the bit of the clamped value, value > 0, when the layer is not in
 * binary mode (pass 0). */
int bbhip_fp32_bit_RealToBinary_Forward(float const *dev_x_buf, int *dev_y_buf, unsigned depth_modulation_size, unsigned frame_modulation_size,
                                        float input_range_lo, float input_range_hi, unsigned point_size, unsigned x_depth_size,
                                        unsigned x_frame_size, unsigned x_frame_stride, unsigned y_frame_stride, int binarize, void *stream);
/* bbcu_fp32_BinaryToReal_Forward, include/bbcu/bbcu.h:1376-1387: y[o][g] = the share of inputs > 0 among the input nodes o, O + o, ...
 * (node_mux_size of them) and the frames g * frame_mux_size ... + frame_mux_size - 1, the count divided by their number as on the host
 * (include/bb/BinaryToReal.h:262-290; the reference's device kernel multiplies by a reciprocal). */
int bbhip_fp32_BinaryToReal_Forward(float const *dev_x_buf, float *dev_y_buf, int node_mux_size, int frame_mux_size, int y_node_size,
                                    int x_frame_stride, int y_frame_size, int y_frame_stride, void *stream);
/* bbcu_bit_fp32_BinaryToReal_Forward, include/bbcu/bbcu.h:1389-1400: packed input, rows of x_frame_stride words */
int bbhip_bit_fp32_BinaryToReal_Forward(int const *dev_x_buf, float *dev_y_buf, int node_mux_size, int frame_mux_size, int y_node_size,
                                        int x_frame_stride, int y_frame_size, int y_frame_stride, void *stream);
/* bbcu_fp32_BinaryToReal_Backward, include/bbcu/bbcu.h:1402-1413: every input that folds into (o, g) receives
 * dy[o][g] * (O / (I * frame_mux_size)) (include/bb/BinaryToReal.h:333-352) */
int bbhip_fp32_BinaryToReal_Backward(float const *dev_dy_buf, float *dev_dx_buf, int node_mux_size, int frame_mux_size, int y_node_size,
                                     int x_frame_stride, int y_frame_size, int y_frame_stride, void *stream);

/* ---- Binarize, HardTanh ---- */
/* bbcu_fp32_Binarize_Forward, include/bbcu/bbcu.h:1223-1234: y = x > binary_th ? binary_high : binary_low (include/bb/Binarize.h:196-213) */
int bbhip_fp32_Binarize_Forward(float const *dev_x_buf, float *dev_y_buf, float binary_th, float binary_low, float binary_high,
                                int node_size, int frame_size, int frame_stride, void *stream);
/* bbcu_fp32_bit_Binarize_Forward, include/bbcu/bbcu.h:1236-1246: the packed bits of x > binary_th (bits past the last frame written as 0) */
int bbhip_fp32_bit_Binarize_Forward(float const *dev_x_buf, int *dev_y_buf, float binary_th, int node_size, int frame_size,
                                    int x_frame_stride, int y_frame_stride, void *stream);
/* bbcu_fp32_HardTanh_Forward, include/bbcu/bbcu.h:1253-1263: x <= limit_min -> limit_min, x >= limit_max -> limit_max
 * (include/bb/HardTanh.h:176-193) */
int bbhip_fp32_HardTanh_Forward(float const *dev_x_buf, float *dev_y_buf, float limit_min, float limit_max, int node_size, int frame_size,
                                int frame_stride, void *stream);
/* bbcu_fp32_HardTanh_Backward, include/bbcu/bbcu.h:1265-1276: dx = dy where limit_min < x < limit_max, else 0; also the backward of
 * Binarize (include/bb/HardTanh.h:253-271, Binarize.h:268-285) */
int bbhip_fp32_HardTanh_Backward(float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, float limit_min, float limit_max,
                                 int node_size, int frame_size, int frame_stride, void *stream);

/* ---- MaxPooling, UpSampling ----
 * Windows of filter_h x filter_w tile the image without overlap, the last ones cut off at the border: output = ceil(input / filter).
 * Bit-exact with the reference's host loops. */
/* bbcu_fp32_MaxPooling_Forward, include/bbcu/bbcu.h:949-964: y = the largest value of the window, argmax = the position of its first
 * occurrence counted in (fy, fx) order over the window's positions inside the image (include/bb/MaxPooling.h:251-284) */
int bbhip_fp32_MaxPooling_Forward(float const *dev_x_buf, float *dev_y_buf, int *dev_argmax_buf, int filter_h_size, int filter_w_size,
                                  int input_w_size, int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size,
                                  int frame_stride, void *stream);
/* bbcu_bit_MaxPooling_Forward, include/bbcu/bbcu.h:966-980: packed rows, y = the OR of the window (bits past the last frame written as 0) */
int bbhip_bit_MaxPooling_Forward(int const *dev_x_buf, int *dev_y_buf, int filter_h_size, int filter_w_size, int input_w_size,
                                 int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size, int frame_stride,
                                 void *stream);
/* bbcu_fp32_MaxPooling_Backward, include/bbcu/bbcu.h:983-998: the recorded position of each window receives dy, the others 0 */
int bbhip_fp32_MaxPooling_Backward(int const *dev_argmax_buf, float const *dev_dy_buf, float *dev_dx_buf, int filter_h_size, int filter_w_size,
                                   int input_w_size, int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size,
                                   int frame_stride, void *stream);
/* bbcu_bit_fp32_MaxPooling_Backward, include/bbcu/bbcu.h:1000-1016: dy goes to the first set input of each window in (fy, fx) order,
 * to none when none is set (include/bb/MaxPooling.h:551-579); x is the packed forward input */
int bbhip_bit_fp32_MaxPooling_Backward(int const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, int filter_h_size, int filter_w_size,
                                       int input_w_size, int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size,
                                       int forward_frame_stride, int backward_frame_stride, void *stream);
/* bbcu_fp32_UpSampling_Forward, include/bbcu/bbcu.h:1024-1037: every input pixel becomes a filter_h x filter_w block, all of it (fill)
 * or only its position (filter_h / 2, filter_w / 2) with zeros around (include/bb/UpSampling.h:223-259) */
int bbhip_fp32_UpSampling_Forward(float const *dev_x_buf, float *dev_y_buf, int input_w_size, int input_h_size, int c_size, int filter_w_size,
                                  int filter_h_size, int fill, int frame_size, int frame_stride, void *stream);
/* bbcu_bit_UpSampling_Forward, include/bbcu/bbcu.h:1039-1052: packed rows of frame_stride words */
int bbhip_bit_UpSampling_Forward(int const *dev_x_buf, int *dev_y_buf, int input_w_size, int input_h_size, int c_size, int filter_w_size,
                                 int filter_h_size, int fill, int frame_size, int frame_stride, void *stream);
/* bbcu_fp32_UpSampling_Backward, include/bbcu/bbcu.h:1055-1068: dx = the sum of dy over the block in (fy, fx) order, or dy at the
 * block's position (filter_h / 2, filter_w / 2) (include/bb/UpSampling.h:321-353) */
int bbhip_fp32_UpSampling_Backward(float const *dev_dy_buf, float *dev_dx_buf, int input_w_size, int input_h_size, int c_size, int filter_w_size,
                                   int filter_h_size, int fill, int frame_size, int frame_stride, void *stream);

/* ---- Shuffle ----
 * bbcu_Shuffle_Forward<T>, include/bbcu/bbcu.h:1194-1204: with x_unit_size = node_size / y_unit_size, output row i * y_unit_size + j is
 * input row j * x_unit_size + i (include/bb/Shuffle.h:166-185).  Rows are frame_stride 32-bit words whatever they hold (fp32 frames or
 * packed bits: the reference's class passes both as int) and are copied whole; node_size must be a multiple of y_unit_size. */
int bbhip_Shuffle_Forward(int const *dev_x_buf, int *dev_y_buf, unsigned int y_unit_size, unsigned int node_size, unsigned int frame_size,
                          unsigned int frame_stride, void *stream);
/* bbcu_Shuffle_Backward<T>, include/bbcu/bbcu.h:1206-1216: input-gradient row i * x_unit_size + j is output-gradient row
 * j * y_unit_size + i (include/bb/Shuffle.h:225-243) */
int bbhip_Shuffle_Backward(int const *dev_dy_buf, int *dev_dx_buf, unsigned int y_unit_size, unsigned int node_size, unsigned int frame_size,
                           unsigned int frame_stride, void *stream);

/* ---- mean squared error ---- */
/* bbcu_fp32_LossMeanSquaredError, include/bbcu/bbcu.h:1487-1500: dy = (y - t) * grad_reduction (the caller passes 2 / (nodes * batch)
 * or 2); dev_loss_buf[s] += the sum over the frames s, s + loss_buf_size, ... and all nodes of (float)(y - t)^2 * loss_reduction in
 * double, squares that are NaN left out as on the host path (include/bb/LossMeanSquaredError.h:150-169).  The caller adds the
 * loss_buf_size entries up.  Sums are taken node ascending within groups of 64 nodes, then groups, then frames: the same bits on
 * every run, and equal to the host's single running sum to rounding of doubles. */
int bbhip_fp32_LossMeanSquaredError(float const *dev_y_buf, float const *dev_t_buf, float *dev_dy_buf, double *dev_loss_buf, int loss_buf_size,
                                    int node_size, int frame_size, int frame_stride, float grad_reduction, double loss_reduction, void *stream);
/* No counterpart in include/bbcu/bbcu.h (the reference computes this metric on the host, include/bb/MetricsMeanSquaredError.h:66-85):
 * dev_accuracy_buf[s] += the sum over the frames s, s + accuracy_buf_size, ... and all nodes of (float)(t - y)^2 / node_size. */
int bbhip_fp32_MetricsMeanSquaredError(float const *dev_y_buf, float const *dev_t_buf, double *dev_accuracy_buf, int accuracy_buf_size,
                                       int node_size, int frame_size, int frame_stride, void *stream);

/* bbcu_LossSoftmaxCrossEntropy<float>, include/bbcu/bbcu.h:1506-1519.  Nodes are [ch][pix]; per frame and pixel softmax over the
 * channels; dev_loss_buf[frame] = sum over pixels and channels with t > 0 of log(softmax + 1e-7) * t_max (t_max = sum of the pixel's
 * targets), dy = (t_max * softmax - t) / t_sum.  The caller passes t_sum = sum of all targets and reports
 * -sum(dev_loss_buf) / t_sum (include/bb/LossSoftmaxCrossEntropy.h:99-125, 159-219).  dy is divided by t_sum as on the host path;
 * the CUDA kernel multiplies by its reciprocal. */
int bbhip_fp32_LossSoftmaxCrossEntropy(float const *dev_y_buf, float const *dev_t_buf, float *dev_dy_buf, double *dev_loss_buf, float t_sum,
                                       int pix_size, int ch_size, int frame_size, int frame_stride, void *stream);
/* bbcu_MetricsCategoricalAccuracy<float>, include/bbcu/bbcu.h:1540-1553: per frame, dev_category_buf = pixels with a positive target,
 * dev_accuracy_buf = those of them whose first largest y sits on a channel with a positive target */
int bbhip_fp32_MetricsCategoricalAccuracy(float const *dev_y_buf, float const *dev_t_buf, int *dev_accuracy_buf, int *dev_category_buf,
                                          int pix_size, int ch_size, int frame_size, int frame_stride, void *stream);

/* ---- StochasticBatchNormalization ----
 * Per node (a row of frames): mean and biased variance of the batch, rstd = 1 / (sqrt(var) + 1e-7),
 * y = ((x - mean) * rstd) * gamma + beta with one scalar gamma and beta for the layer
 * (include/bb/StochasticBatchNormalization.h:535-597).  Sums are taken in a fixed tree order: results are the same on every
 * run and agree with the reference's frame-order sums to rounding. */
/* bbcu_fp32_StochasticBatchNormalization_ForwardTraining, include/bbcu/bbcu.h:883-898: also writes the batch statistics and
 * updates running = running * momentum + batch * (1 - momentum) */
int bbhip_fp32_StochasticBatchNormalization_ForwardTraining(float const *dev_x_buf, float *dev_y_buf, float *dev_mean_buf, float *dev_rstd_buf,
                                                            float *dev_running_mean_buf, float *dev_running_var_buf, float gamma, float beta,
                                                            float momentum, int node_size, int frame_size, int frame_stride, void *stream);
/* bbcu_fp32_StochasticBatchNormalization_ReForward, include/bbcu/bbcu.h:900-912: the output again from stored batch statistics */
int bbhip_fp32_StochasticBatchNormalization_ReForward(float const *dev_x_buf, float *dev_y_buf, float const *dev_mean_buf,
                                                      float const *dev_rstd_buf, float gamma, float beta, int node_size, int frame_size,
                                                      int frame_stride, void *stream);
/* bbcu_fp32_StochasticBatchNormalization_ForwardInference, include/bbcu/bbcu.h:914-926: mean = running mean,
 * rstd = 1 / (sqrt(running var) + 1e-7) */
int bbhip_fp32_StochasticBatchNormalization_ForwardInference(float const *dev_x_buf, float *dev_y_buf, float const *dev_running_mean_buf,
                                                             float const *dev_running_var_buf, float gamma, float beta, int node_size,
                                                             int frame_size, int frame_stride, void *stream);
/* bbcu_fp32_StochasticBatchNormalization_Backward, include/bbcu/bbcu.h:928-942 (host loop: StochasticBatchNormalization.h:815-851);
 * dev_x_buf rows are x_frame_stride apart, dy and dx rows frame_stride */
int bbhip_fp32_StochasticBatchNormalization_Backward(float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf,
                                                     float const *dev_mean_buf, float const *dev_rstd_buf, float gamma,
                                                     float reciprocal_frame_size, int node_size, int frame_size, int frame_stride,
                                                     int x_frame_stride, void *stream);

/* ---- StochasticLut ---- */
/* bbcu_fp32_StochasticLut_Forward<N>, include/bbcu/bbcu.h:667-681 */
int bbhip_fp32_StochasticLut_Forward(int n, float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index,
                                     float const *dev_W, int node_size, int frame_size, int frame_stride,
                                     int input_binary, int lut_binarize, float unbinarize_bias, void *stream);
/* No single counterpart in the reference: its model class clamps the table in place and then calls the forward entry
 * (m_W->Clamp_inplace(0, 1), include/bb/StochasticLutN.h:451, i.e. bbcu_fp32_Vector_clamp followed by
 * bbcu_fp32_StochasticLut_Forward<N>).  This entry does both — dev_W is clamped to [w_lo, w_hi] in place by the launch that
 * prepares the tables, then the forward pass runs on the clamped table: the same results as
 * bbhip_fp32_Vector_clamp(dev_W, dev_W, w_lo, w_hi, node_size << n) + bbhip_fp32_StochasticLut_Forward, one launch fewer. */
int bbhip_fp32_StochasticLut_ForwardClampW(int n, float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index,
                                           float *dev_W, int node_size, int frame_size, int frame_stride,
                                           int input_binary, int lut_binarize, float unbinarize_bias,
                                           float w_lo, float w_hi, void *stream);
/* No counterpart in the reference.  bbhip_fp32_StochasticLut_Forward for callers that cannot allocate device memory — code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc: same arguments and results, but the
 * tables that the kernels read come from a fixed 8 MiB block inside the library (one per GPU, held until the process
 * ends) instead of the growing arena, and the call never calls hipMalloc, hipFree or any allocating routine.  Limit:
 * node_size * 2^n * 4 bytes (twice that with input_binary) must fit the block — 32768 nodes (16384 with input_binary)
 * at n = 6; larger layers are rejected with a message.  bbhip_HintInputNodeSize is ignored and the kernel timer does not
 * record this entry.  All calls on a GPU share the block: calls that overlap on one GPU (two streams, two threads) race. */
int bbhip_fp32_StochasticLut_Forward_NoAlloc(int n, float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index,
                                             float const *dev_W, int node_size, int frame_size, int frame_stride,
                                             int input_binary, int lut_binarize, float unbinarize_bias, void *stream);
/* bbcu_bit_fp32_StochasticLut_Forward<N>, include/bbcu/bbcu.h:683-697 */
int bbhip_bit_fp32_StochasticLut_Forward(int n, int const *dev_x_buf, float *dev_y_buf, int const *dev_input_index,
                                         float const *dev_W, int node_size, int frame_size, int frame_stride,
                                         int bin_frame_stride, int lut_binarize, float unbinarize_bias, void *stream);
/* bbcu_bit_bit_fp32_StochasticLut_Forward<N>, include/bbcu/bbcu.h:699-712 */
int bbhip_bit_bit_fp32_StochasticLut_Forward(int n, int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index,
                                             float const *dev_W, int node_size, int frame_size, int frame_stride,
                                             int lut_binarize, float unbinarize_bias, void *stream);
/* bbcu_fp32_StochasticLut_Backward<N>, include/bbcu/bbcu.h:715-737 */
int bbhip_fp32_StochasticLut_Backward(int n, float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf,
                                      float *dev_dx_tmp, int const *dev_input_index, int const *dev_reverse_index,
                                      float const *dev_W, float *dev_dW, int reverse_index_stride,
                                      int input_node_size, int output_node_size, int frame_size, int frame_stride,
                                      int tmp_frame_size, int tmp_frame_stride, int input_binary, int lut_binarize,
                                      float unbinarize_bias, void *stream);
/* bbcu_bit_fp32_StochasticLut_Backward<N>, include/bbcu/bbcu.h:739-761 */
int bbhip_bit_fp32_StochasticLut_Backward(int n, int const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf,
                                          float *dev_dx_tmp, int const *dev_input_index, int const *dev_reverse_index,
                                          float const *dev_W, float *dev_dW, int reverse_index_stride,
                                          int input_node_size, int output_node_size, int frame_size, int frame_stride,
                                          int bin_frame_stride, int tmp_frame_size, int tmp_frame_stride,
                                          int lut_binarize, float unbinarize_bias, void *stream);

/* ---- DifferentiableLut (LUT fused with per-node batch normalisation and binarize / hard-tanh) ---- */
/* bbcu_fp32_DifferentiableLutN_ForwardTraining<N>, include/bbcu/bbcu.h:518-539 */
int bbhip_fp32_DifferentiableLutN_ForwardTraining(int n, float const *dev_x_buf, float *dev_y_buf,
        int const *dev_input_index, float const *dev_W, float *dev_mean_buf, float *dev_rstd_buf,
        float *dev_running_mean_buf, float *dev_running_var_buf, float gamma, float beta, float momentum,
        float unbinarize_bias, int node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode,
        void *stream);
/* bbcu_bit_fp32_DifferentiableLutN_ForwardTraining<N>, include/bbcu/bbcu.h:541-561 */
int bbhip_bit_fp32_DifferentiableLutN_ForwardTraining(int n, int const *dev_x_buf, int *dev_y_buf,
        int const *dev_input_index, float const *dev_W, float *dev_mean_buf, float *dev_rstd_buf,
        float *dev_running_mean_buf, float *dev_running_var_buf, float gamma, float beta, float momentum,
        float unbinarize_bias, int node_size, int frame_size, int frame_stride, int lut_binarize, void *stream);
/* No single counterpart in the reference: its model class clamps the table in place before the first forward pass after a
 * backward pass (m_W->Clamp_inplace(0, 1), include/bb/DifferentiableLutN.h:605-608) and then calls the forward entry.  These two
 * do both, like bbhip_fp32_StochasticLut_ForwardClampW: dev_W is clamped to [w_lo, w_hi] in place by the launch that prepares
 * the tables, and the pass runs on the clamped table; all other arguments and results as in the entries above. */
int bbhip_fp32_DifferentiableLutN_ForwardTrainingClampW(int n, float const *dev_x_buf, float *dev_y_buf,
        int const *dev_input_index, float *dev_W, float *dev_mean_buf, float *dev_rstd_buf,
        float *dev_running_mean_buf, float *dev_running_var_buf, float gamma, float beta, float momentum,
        float unbinarize_bias, int node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode,
        float w_lo, float w_hi, void *stream);
int bbhip_bit_fp32_DifferentiableLutN_ForwardTrainingClampW(int n, int const *dev_x_buf, int *dev_y_buf,
        int const *dev_input_index, float *dev_W, float *dev_mean_buf, float *dev_rstd_buf,
        float *dev_running_mean_buf, float *dev_running_var_buf, float gamma, float beta, float momentum,
        float unbinarize_bias, int node_size, int frame_size, int frame_stride, int lut_binarize,
        float w_lo, float w_hi, void *stream);
/* bbcu_fp32_DifferentiableLutN_ForwardInference<N>, include/bbcu/bbcu.h:563-581
 * (rstd = 1/sqrt(running_var) and the hard-tanh clip follow the reference's CPU path, include/bb/DifferentiableLutN.h:866-897) */
int bbhip_fp32_DifferentiableLutN_ForwardInference(int n, float const *dev_x_buf, float *dev_y_buf,
        int const *dev_input_index, float const *dev_W, float const *dev_running_mean_buf,
        float const *dev_running_var_buf, float gamma, float beta, float unbinarize_bias,
        int node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode, void *stream);
/* bbcu_bit_fp32_DifferentiableLutN_ForwardInference<N>, include/bbcu/bbcu.h:583-600 */
int bbhip_bit_fp32_DifferentiableLutN_ForwardInference(int n, int const *dev_x_buf, int *dev_y_buf,
        int const *dev_input_index, float const *dev_W, float const *dev_running_mean_buf,
        float const *dev_running_var_buf, float gamma, float beta, float unbinarize_bias,
        int node_size, int frame_size, int frame_stride, int lut_binarize, void *stream);
/* bbcu_fp32_DifferentiableLutN_Backward<N>, include/bbcu/bbcu.h:602-630 */
int bbhip_fp32_DifferentiableLutN_Backward(int n, float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf,
        float *dev_dx_tmp, int const *dev_input_index, int const *dev_reverse_index, float const *dev_W,
        float *dev_dW, float const *dev_mean_buf, float const *dev_rstd_buf, float *dev_dmean_tmp,
        float *dev_dvar_tmp, float gamma, float beta, float unbinarize_bias, int reverse_index_stride,
        int input_node_size, int output_node_size, int frame_size, int frame_stride, int tmp_frame_size,
        int tmp_frame_stride, int lut_binarize, int binary_mode, void *stream);
/* bbcu_bit_fp32_DifferentiableLutN_Backward<N>, include/bbcu/bbcu.h:632-660 */
int bbhip_bit_fp32_DifferentiableLutN_Backward(int n, int const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf,
        float *dev_dx_tmp, int const *dev_input_index, int const *dev_reverse_index, float const *dev_W,
        float *dev_dW, float const *dev_mean_buf, float const *dev_rstd_buf, float *dev_dmean_tmp,
        float *dev_dvar_tmp, float gamma, float beta, float unbinarize_bias, int reverse_index_stride,
        int input_node_size, int output_node_size, int frame_size, int frame_stride, int x_frame_stride,
        int tmp_frame_size, int tmp_frame_stride, int lut_binarize, void *stream);
/* DifferentiableLutN<N,float>::Forward without batch-norm on the reference's CPU path binarizes the output in binary
 * mode (include/bb/DifferentiableLutN.h:994-1002); its CUDA path calls bbcu_fp32_StochasticLut_Forward, which only clips.
 * This entry point gives the CPU behaviour: y = binary_mode ? (LUT > 0.5) : clip(LUT, 0, 1). */
int bbhip_fp32_DifferentiableLutN_ForwardNoBn(int n, float const *dev_x_buf, float *dev_y_buf,
        int const *dev_input_index, float const *dev_W, float unbinarize_bias,
        int node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode, void *stream);

/* ---- BinaryLut6 ---- */
/* bbcu_bit_BinatyLut6_Forward [sic], include/bbcu/bbcu.h:285-295. Bits of the last word beyond frame_size are written as 0. */
int bbhip_bit_BinaryLut6_Forward(int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, int const *dev_table,
                                 int node_size, int frame_size, int frame_stride, void *stream);

/* BinaryLutN<N> for n = 2 .. 6 on packed bits.  The reference has a device entry for n = 6 only (above; n = 6 is forwarded to it) and runs
 * the other widths in its generic host loop (include/bb/BinaryLutN.h:436-463), which is what this entry computes: input k of a node is
 * bit k of the table index, dev_table is [node_size][1] words for n <= 5 (entry i = bit i), [node_size][2] for n = 6.  With it a layer
 * trained at any width (StochasticLutN / DifferentiableLutN, n = 2 .. 6) can be tabulated and run packed on the device. */
int bbhip_bit_BinaryLutN_Forward(int n, int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, int const *dev_table,
                                 int node_size, int frame_size, int frame_stride, void *stream);

#ifdef __cplusplus
}
#endif

#endif  /* BBHIP_H_ */
