/*
 * bbcu_hip_binding.h — BinaryBrain's device entry points under their own names, forwarding to the C ABI of bbhip.h.
 *
 * BinaryBrain's layers call functions declared in the reference's include/bbcu/bbcu.h: plain functions, and C++ function
 * templates on the LUT width N (default 6, instantiated for 2..6) or on the element type.  Every function below has the
 * reference's name, parameter list and defaults (cudaStream_t streamId = 0 last); the file:line of the declaration it
 * stands in for is cited on each.  The LUT width moves from the template parameter to the first argument of the C ABI,
 * the stream is passed on as an opaque handle.  With this header included in place of those declarations (and the
 * library linked instead of libbbcu), include/bb/StochasticLutN.h, DifferentiableLutN.h, BinaryLutN.h and the layers
 * around them compile against it unchanged.
 *
 * Return value: 0, as in the reference (whose callers never look at it).  Where the reference prints, waits on stdin and
 * exits on a failed launch (include/bbcu/bbcu_util.h:17-36), these wrappers throw std::runtime_error with the library's
 * message.
 */
#ifndef BBCU_HIP_BINDING_H_
#define BBCU_HIP_BINDING_H_

#include <stddef.h>
#include <stdexcept>
#include <type_traits>

#include "bbhip.h"

#ifndef BBCU_HIP_BINDING_NO_STREAM_TYPE
typedef void *cudaStream_t;         /* only ever an opaque handle in these signatures (define the macro where a real one exists) */
#endif

#define BBCU_HIP_CALL(expr) do { if ((expr) != 0) { throw std::runtime_error(bbhip_GetLastErrorString()); } } while (0)

/* ---- device manager, include/bbcu/bbcu.h:49-55 ---- */
inline int  bbcu_GetDeviceCount(void)       { return bbhip_GetDeviceCount(); }
inline int  bbcu_GetDevice(void)            { return bbhip_GetDevice(); }
inline void bbcu_SetDevice(int device)      { bbhip_SetDevice(device); }
inline void bbcu_SetHostOnly(bool hostOnly) { bbhip_SetHostOnly(hostOnly ? 1 : 0); }
inline bool bbcu_IsHostOnly(void)           { return bbhip_IsHostOnly() != 0; }
inline bool bbcu_IsDeviceAvailable(void)    { return bbhip_IsDeviceAvailable() != 0; }

/* ---- local heap, include/bbcu/bbcu.h:63-67 ---- */
inline void  *bbcu_LocalHeap_Malloc(size_t size)        { return bbhip_LocalHeap_Malloc(size); }
inline void   bbcu_LocalHeap_Free(void *ptr)            { bbhip_LocalHeap_Free(ptr); }
inline size_t bbcu_LocalHeap_GetMaxAllocSize(void)      { return bbhip_LocalHeap_GetMaxAllocSize(); }
inline size_t bbcu_LocalHeap_GetAllocatedSize(void)     { return bbhip_LocalHeap_GetAllocatedSize(); }
inline void   bbcu_LocalHeap_GarbageCollect(void)       { bbhip_LocalHeap_GarbageCollect(); }

/* ---- memory helpers of namespace bbcu, include/bbcu/bbcu_util.h:89-134; kind as cudaMemcpyKind: 1 host to device,
 * 2 device to host, 3 device to device ---- */
namespace bbcu {
inline void   Malloc(void **ptr, size_t size)                           { BBCU_HIP_CALL(bbhip_Malloc(ptr, size == 0 ? 4 : size)); }
inline void   Free(void *ptr)                                           { BBCU_HIP_CALL(bbhip_Free(ptr)); }
inline size_t GetMaxAllocSize(void)                                     { return bbhip_LocalHeap_GetMaxAllocSize(); }
inline void   MallocHost(void **ptr, size_t size, unsigned int = 0)     { BBCU_HIP_CALL(bbhip_MallocHost(ptr, size)); }
inline void   FreeHost(void *ptr)                                       { BBCU_HIP_CALL(bbhip_FreeHost(ptr)); }
inline void   Memcpy(void *dst, const void *src, size_t count, int kind) { if (count > 0) { BBCU_HIP_CALL(bbhip_Memcpy(dst, src, count, kind)); } }
}  // namespace bbcu

/* ---- vector operations, include/bbcu/bbcu.h:89-198 ---- */
inline int bbcu_fp32_Vector_set(float *dev_dst, float a, int size, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_fp32_Vector_set(dev_dst, a, size, streamId)); return 0; }
inline int bbcu_fp32_Vector_add_ex(float *dev_dst, const float *dev_src0, const float *dev_src1, float a, float b, float c, int size,
                                   cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_fp32_Vector_add_ex(dev_dst, dev_src0, dev_src1, a, b, c, size, streamId)); return 0; }
inline int bbcu_fp32_Vector_mul_ex(float *dev_dst, const float *dev_src0, const float *dev_src1, float a, float b, int size,
                                   cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_fp32_Vector_mul_ex(dev_dst, dev_src0, dev_src1, a, b, size, streamId)); return 0; }
inline int bbcu_fp32_Vector_div_ex(float *dev_dst, float const *dev_src0, float const *dev_src1, float a, float b, float c, float d,
                                   int size, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_fp32_Vector_div_ex(dev_dst, dev_src0, dev_src1, a, b, c, d, size, streamId)); return 0; }
inline int bbcu_fp32_Vector_sqrt(float *dev_dst, float const *dev_src, int size, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_fp32_Vector_sqrt(dev_dst, dev_src, size, streamId)); return 0; }
inline int bbcu_fp32_Vector_exp(float *dev_dst, float const *dev_src, int size, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_fp32_Vector_exp(dev_dst, dev_src, size, streamId)); return 0; }
inline int bbcu_fp32_Vector_min(float *dev_dst, float const *dev_src0, float const *dev_src1, int size, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_fp32_Vector_min(dev_dst, dev_src0, dev_src1, size, streamId)); return 0; }
inline int bbcu_fp32_Vector_min_v(float *dev_dst, float const *dev_src, float a, int size, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_fp32_Vector_min_v(dev_dst, dev_src, a, size, streamId)); return 0; }
inline int bbcu_fp32_Vector_max(float *dev_dst, float const *dev_src0, float const *dev_src1, int size, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_fp32_Vector_max(dev_dst, dev_src0, dev_src1, size, streamId)); return 0; }
inline int bbcu_fp32_Vector_max_v(float *dev_dst, float const *dev_src, float a, int size, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_fp32_Vector_max_v(dev_dst, dev_src, a, size, streamId)); return 0; }
inline int bbcu_fp32_Vector_clamp(float *dev_dst, float const *dev_src, float lo, float hi, int size, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_fp32_Vector_clamp(dev_dst, dev_src, lo, hi, size, streamId)); return 0; }

/* ---- bbcu_ConvBitToReal<T>, include/bbcu/bbcu.h:246-258 (T = float) ---- */
template <typename T = float>
int bbcu_ConvBitToReal(int const *dev_x_buf, T *dev_y_buf, T value0, T value1, int node_size, int frame_size, int x_frame_stride,
                       int y_frame_stride, cudaStream_t streamId = 0)
{
    static_assert(std::is_same<T, float>::value, "fp32 frames");
    BBCU_HIP_CALL(bbhip_fp32_ConvBitToReal(dev_x_buf, dev_y_buf, value0, value1, node_size, frame_size, x_frame_stride, y_frame_stride, streamId));
    return 0;
}

/* ---- bbcu_bit_BinatyLut6_Forward [sic], include/bbcu/bbcu.h:285-295 ---- */
inline int bbcu_bit_BinatyLut6_Forward(int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, int const *dev_table,
                                       int node_size, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_bit_BinaryLut6_Forward(dev_x_buf, dev_y_buf, dev_input_index, dev_table, node_size, frame_size, frame_stride, streamId)); return 0; }

/* ---- AverageLut, include/bbcu/bbcu.h:321-361 (T = float).  Without binarize_output the forward entry writes sum * (1 / n), as the
 * CUDA kernel of this name does (cuda/AverageLut.cu:46-54); the host loop's plain sum is bbhip_fp32_AverageLut_ForwardSum ---- */
template <typename T>
int bbcu_AverageLut_Forward(T const *dev_x_buf, T *dev_y_buf, int const *dev_input_index, int n, int node_size, int frame_size,
                            int frame_stride, bool binarize_input, bool binarize_output, cudaStream_t streamId = 0)
{
    static_assert(std::is_same<T, float>::value, "fp32 frames");
    BBCU_HIP_CALL(bbhip_fp32_AverageLut_Forward(dev_x_buf, dev_y_buf, dev_input_index, n, node_size, frame_size, frame_stride,
                                                binarize_input ? 1 : 0, binarize_output ? 1 : 0, streamId));
    return 0;
}
inline int bbcu_bit_AverageLut_Forward(int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, int n, int node_size,
                                       int frame_size, int frame_stride, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_bit_AverageLut_Forward(dev_x_buf, dev_y_buf, dev_input_index, n, node_size, frame_size, frame_stride, streamId)); return 0; }
template <typename T>
int bbcu_AverageLut_Backward(T const *dev_dy_buf, T *dev_dx_buf, int const *dev_input_index, int n, int input_node_size,
                             int output_node_size, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    static_assert(std::is_same<T, float>::value, "fp32 frames");
    BBCU_HIP_CALL(bbhip_fp32_AverageLut_Backward(dev_dy_buf, dev_dx_buf, dev_input_index, n, input_node_size, output_node_size, frame_size,
                                                 frame_stride, streamId));
    return 0;
}

/* ---- DifferentiableLut, include/bbcu/bbcu.h:518-660 ---- */
template <int N = 6>
int bbcu_fp32_DifferentiableLutN_ForwardTraining(float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index, float const *dev_W,
        float *dev_mean_buf, float *dev_rstd_buf, float *dev_running_mean_buf, float *dev_running_var_buf, float gamma, float beta,
        float momentum, float unbinarize_bias, int node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode,
        cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_DifferentiableLutN_ForwardTraining(N, dev_x_buf, dev_y_buf, dev_input_index, dev_W, dev_mean_buf, dev_rstd_buf,
            dev_running_mean_buf, dev_running_var_buf, gamma, beta, momentum, unbinarize_bias, node_size, frame_size, frame_stride,
            lut_binarize, binary_mode, streamId));
    return 0;
}
template <int N = 6>
int bbcu_bit_fp32_DifferentiableLutN_ForwardTraining(int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, float const *dev_W,
        float *dev_mean_buf, float *dev_rstd_buf, float *dev_running_mean_buf, float *dev_running_var_buf, float gamma, float beta,
        float momentum, float unbinarize_bias, int node_size, int frame_size, int frame_stride, int lut_binarize, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_bit_fp32_DifferentiableLutN_ForwardTraining(N, dev_x_buf, dev_y_buf, dev_input_index, dev_W, dev_mean_buf, dev_rstd_buf,
            dev_running_mean_buf, dev_running_var_buf, gamma, beta, momentum, unbinarize_bias, node_size, frame_size, frame_stride,
            lut_binarize, streamId));
    return 0;
}
template <int N = 6>
int bbcu_fp32_DifferentiableLutN_ForwardInference(float const *dev_x_buf, float *dev_y_buf, int const *dev_input_index, float const *dev_W,
        float const *running_mean_buf, float const *running_var_buf, float gamma, float beta, float unbinarize_bias, int node_size,
        int frame_size, int frame_stride, int lut_binarize, int binary_mode, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_DifferentiableLutN_ForwardInference(N, dev_x_buf, dev_y_buf, dev_input_index, dev_W, running_mean_buf,
            running_var_buf, gamma, beta, unbinarize_bias, node_size, frame_size, frame_stride, lut_binarize, binary_mode, streamId));
    return 0;
}
template <int N = 6>
int bbcu_bit_fp32_DifferentiableLutN_ForwardInference(int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, float const *dev_W,
        float const *running_mean_buf, float const *running_var_buf, float gamma, float beta, float unbinarize_bias, int node_size,
        int frame_size, int frame_stride, int lut_binarize, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_bit_fp32_DifferentiableLutN_ForwardInference(N, dev_x_buf, dev_y_buf, dev_input_index, dev_W, running_mean_buf,
            running_var_buf, gamma, beta, unbinarize_bias, node_size, frame_size, frame_stride, lut_binarize, streamId));
    return 0;
}
template <int N = 6>
int bbcu_fp32_DifferentiableLutN_Backward(float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, float *dev_dx_tmp,
        int const *dev_input_index, int const *dev_reverse_index, float const *dev_W, float *dev_dW, float const *dev_mean_buf,
        float const *dev_rstd_buf, float *dev_dmean_tmp, float *dev_dvar_tmp, float gamma, float beta, float unbinarize_bias,
        int reverse_index_stride, int input_node_size, int output_node_size, int frame_size, int frame_stride, int tmp_frame_size,
        int tmp_frame_stride, int lut_binarize, int binary_mode, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_DifferentiableLutN_Backward(N, dev_x_buf, dev_dy_buf, dev_dx_buf, dev_dx_tmp, dev_input_index, dev_reverse_index,
            dev_W, dev_dW, dev_mean_buf, dev_rstd_buf, dev_dmean_tmp, dev_dvar_tmp, gamma, beta, unbinarize_bias, reverse_index_stride,
            input_node_size, output_node_size, frame_size, frame_stride, tmp_frame_size, tmp_frame_stride, lut_binarize, binary_mode, streamId));
    return 0;
}
template <int N = 6>
int bbcu_bit_fp32_DifferentiableLutN_Backward(int const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, float *dev_dx_tmp,
        int const *dev_input_index, int const *dev_reverse_index, float const *dev_W, float *dev_dW, float const *dev_mean_buf,
        float const *dev_rstd_buf, float *dev_dmean_tmp, float *dev_dvar_tmp, float gamma, float beta, float unbinarize_bias,
        int reverse_index_stride, int input_node_size, int output_node_size, int frame_size, int frame_stride, int x_frame_stride,
        int tmp_frame_size, int tmp_frame_stride, int lut_binarize, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_bit_fp32_DifferentiableLutN_Backward(N, dev_x_buf, dev_dy_buf, dev_dx_buf, dev_dx_tmp, dev_input_index,
            dev_reverse_index, dev_W, dev_dW, dev_mean_buf, dev_rstd_buf, dev_dmean_tmp, dev_dvar_tmp, gamma, beta, unbinarize_bias,
            reverse_index_stride, input_node_size, output_node_size, frame_size, frame_stride, x_frame_stride, tmp_frame_size,
            tmp_frame_stride, lut_binarize, streamId));
    return 0;
}

/* ---- StochasticLut, include/bbcu/bbcu.h:667-761 ---- */
template <int N = 6>
int bbcu_fp32_StochasticLut_Forward(const float *dev_x_buf, float *dev_y_buf, int const *dev_input_index, float const *dev_W, int node_size,
        int frame_size, int frame_stride, int input_binary, int lut_binarize, float unbinarize_bias, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_StochasticLut_Forward(N, dev_x_buf, dev_y_buf, dev_input_index, dev_W, node_size, frame_size, frame_stride,
                                                   input_binary, lut_binarize, unbinarize_bias, streamId));
    return 0;
}
template <int N = 6>
int bbcu_bit_fp32_StochasticLut_Forward(int const *dev_x_buf, float *dev_y_buf, int const *dev_input_index, float const *dev_W, int node_size,
        int frame_size, int frame_stride, int bin_frame_stride, int lut_binarize, float unbinarize_bias, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_bit_fp32_StochasticLut_Forward(N, dev_x_buf, dev_y_buf, dev_input_index, dev_W, node_size, frame_size, frame_stride,
                                                       bin_frame_stride, lut_binarize, unbinarize_bias, streamId));
    return 0;
}
template <int N = 6>
int bbcu_bit_bit_fp32_StochasticLut_Forward(int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, float const *dev_W, int node_size,
        int frame_size, int frame_stride, int lut_binarize, float unbinarize_bias, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_bit_bit_fp32_StochasticLut_Forward(N, dev_x_buf, dev_y_buf, dev_input_index, dev_W, node_size, frame_size, frame_stride,
                                                           lut_binarize, unbinarize_bias, streamId));
    return 0;
}
template <int N = 6>
int bbcu_fp32_StochasticLut_Backward(float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, float *dev_dx_tmp,
        int const *dev_input_index, int const *dev_reverse_index, float const *dev_W, float *dev_dW, int reverse_index_stride,
        int input_node_size, int output_node_size, int frame_size, int frame_stride, int tmp_frame_size, int tmp_frame_stride,
        int input_binary, int lut_binarize, float unbinarize_bias, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_StochasticLut_Backward(N, dev_x_buf, dev_dy_buf, dev_dx_buf, dev_dx_tmp, dev_input_index, dev_reverse_index, dev_W,
            dev_dW, reverse_index_stride, input_node_size, output_node_size, frame_size, frame_stride, tmp_frame_size, tmp_frame_stride,
            input_binary, lut_binarize, unbinarize_bias, streamId));
    return 0;
}
template <int N = 6>
int bbcu_bit_fp32_StochasticLut_Backward(int const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, float *dev_dx_tmp,
        int const *dev_input_index, int const *dev_reverse_index, float const *dev_W, float *dev_dW, int reverse_index_stride,
        int input_node_size, int output_node_size, int frame_size, int frame_stride, int bin_frame_stride, int tmp_frame_size,
        int tmp_frame_stride, int lut_binarize, float unbinarize_bias, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_bit_fp32_StochasticLut_Backward(N, dev_x_buf, dev_dy_buf, dev_dx_buf, dev_dx_tmp, dev_input_index, dev_reverse_index,
            dev_W, dev_dW, reverse_index_stride, input_node_size, output_node_size, frame_size, frame_stride, bin_frame_stride,
            tmp_frame_size, tmp_frame_stride, lut_binarize, unbinarize_bias, streamId));
    return 0;
}

/* ---- MaxLut, include/bbcu/bbcu.h:364-427 (T = float).  The running maximum starts at -1, as in the reference's host loop
 * (include/bb/MaxLut.h:293-318), not at the lowest float of its device kernel: outputs are never below -1. ---- */
template <typename T>
int bbcu_MaxLut_Forward(T const *dev_x_buf, T *dev_y_buf, int const *dev_input_index, int n, int node_size, int frame_size,
                        int frame_stride, bool binarize_input, bool binarize_output, cudaStream_t streamId = 0)
{
    static_assert(std::is_same<T, float>::value, "the library holds the fp32 instantiation");
    BBCU_HIP_CALL(bbhip_fp32_MaxLut_Forward(dev_x_buf, dev_y_buf, dev_input_index, n, node_size, frame_size, frame_stride,
                                            binarize_input ? 1 : 0, binarize_output ? 1 : 0, streamId));
    return 0;
}
inline int bbcu_bit_MaxLut_Forward(int const *dev_x_buf, int *dev_y_buf, int const *dev_input_index, int n, int node_size,
                                   int frame_size, int frame_stride, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_bit_MaxLut_Forward(dev_x_buf, dev_y_buf, dev_input_index, n, node_size, frame_size, frame_stride, streamId)); return 0; }
template <typename T>
int bbcu_MaxLut_Backward(T const *dev_x_buf, T const *dev_dy_buf, T *dev_dx_buf, int const *dev_input_index, int n, int input_node_size,
                         int output_node_size, int frame_size, int frame_stride, bool binarize_input, cudaStream_t streamId = 0)
{
    static_assert(std::is_same<T, float>::value, "the library holds the fp32 instantiation");
    BBCU_HIP_CALL(bbhip_fp32_MaxLut_Backward(dev_x_buf, dev_dy_buf, dev_dx_buf, dev_input_index, n, input_node_size, output_node_size, frame_size,
                                             frame_stride, binarize_input ? 1 : 0, streamId));
    return 0;
}
template <typename T>
int bbcu_bit_MaxLut_Backward(int const *dev_x_buf, T const *dev_dy_buf, T *dev_dx_buf, int const *dev_input_index, int n, int input_node_size,
                             int output_node_size, int frame_size, int x_frame_stride, int dy_frame_stride, cudaStream_t streamId = 0)
{
    static_assert(std::is_same<T, float>::value, "the library holds the fp32 instantiation");
    BBCU_HIP_CALL(bbhip_bit_fp32_MaxLut_Backward(dev_x_buf, dev_dy_buf, dev_dx_buf, dev_input_index, n, input_node_size, output_node_size,
                                                 frame_size, x_frame_stride, dy_frame_stride, streamId));
    return 0;
}

/* ---- LossMeanSquaredError, include/bbcu/bbcu.h:1487-1500 ---- */
inline int bbcu_fp32_LossMeanSquaredError(const float *dev_y_buf, const float *dev_t_buf, float *dev_dy_buf, double *dev_loss_buf,
        int loss_buf_size, int node_size, int frame_size, int frame_stride, float grad_reduction, double loss_reduction,
        cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_LossMeanSquaredError(dev_y_buf, dev_t_buf, dev_dy_buf, dev_loss_buf, loss_buf_size, node_size, frame_size,
                                                  frame_stride, grad_reduction, loss_reduction, streamId));
    return 0;
}

/* ---- StochasticMaxPooling2x2, include/bbcu/bbcu.h:768-796 ---- */
inline int bbcu_fp32_StochasticMaxPooling2x2_Forward(float const *dev_x_buf, float *dev_y_buf, int input_w_size, int input_h_size,
        int output_w_size, int output_h_size, int c_size, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_StochasticMaxPooling2x2_Forward(dev_x_buf, dev_y_buf, input_w_size, input_h_size, output_w_size, output_h_size,
                                                             c_size, frame_size, frame_stride, streamId));
    return 0;
}
inline int bbcu_fp32_StochasticMaxPooling2x2_Backward(float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, int input_w_size,
        int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_StochasticMaxPooling2x2_Backward(dev_x_buf, dev_dy_buf, dev_dx_buf, input_w_size, input_h_size, output_w_size,
                                                              output_h_size, c_size, frame_size, frame_stride, streamId));
    return 0;
}

/* ---- StochasticBatchNormalization, include/bbcu/bbcu.h:883-942 ---- */
inline int bbcu_fp32_StochasticBatchNormalization_ForwardTraining(float const *dev_x_buf, float *dev_y_buf, float *dev_mean_buf,
        float *dev_rstd_buf, float *dev_running_mean_buf, float *dev_running_var_buf, float gamma, float beta, float momentum,
        int node_size, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_StochasticBatchNormalization_ForwardTraining(dev_x_buf, dev_y_buf, dev_mean_buf, dev_rstd_buf, dev_running_mean_buf,
                                                                          dev_running_var_buf, gamma, beta, momentum, node_size, frame_size,
                                                                          frame_stride, streamId));
    return 0;
}
inline int bbcu_fp32_StochasticBatchNormalization_ReForward(float const *dev_x_buf, float *dev_y_buf, float const *dev_mean_buf,
        float const *dev_rstd_buf, float gamma, float beta, int node_size, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_StochasticBatchNormalization_ReForward(dev_x_buf, dev_y_buf, dev_mean_buf, dev_rstd_buf, gamma, beta, node_size,
                                                                    frame_size, frame_stride, streamId));
    return 0;
}
inline int bbcu_fp32_StochasticBatchNormalization_ForwardInference(float const *dev_x_buf, float *dev_y_buf, float const *dev_running_mean_buf,
        float const *dev_running_var_buf, float gamma, float beta, int node_size, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_StochasticBatchNormalization_ForwardInference(dev_x_buf, dev_y_buf, dev_running_mean_buf, dev_running_var_buf, gamma,
                                                                           beta, node_size, frame_size, frame_stride, streamId));
    return 0;
}
inline int bbcu_fp32_StochasticBatchNormalization_Backward(float const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf,
        float const *dev_mean_buf, float const *dev_rstd_buf, float gamma, float reciprocal_frame_size, int node_size, int frame_size,
        int frame_stride, int x_frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_StochasticBatchNormalization_Backward(dev_x_buf, dev_dy_buf, dev_dx_buf, dev_mean_buf, dev_rstd_buf, gamma,
                                                                   reciprocal_frame_size, node_size, frame_size, frame_stride, x_frame_stride,
                                                                   streamId));
    return 0;
}

/* ---- RealToBinary / BinaryToReal, include/bbcu/bbcu.h:1337-1413 ---- */
template <typename T = float>
inline int bbcu_RealToBinary_Forward(T const *dev_x_buf, T *dev_y_buf, unsigned int depth_modulation_size, unsigned int frame_modulation_size,
        T input_range_lo, T input_range_hi, unsigned int point_size, unsigned int x_depth_size, unsigned int x_frame_size,
        unsigned int x_frame_stride, unsigned int y_frame_stride, bool binarize, cudaStream_t streamId = 0)
{
    static_assert(sizeof(T) == sizeof(float), "the reference instantiates this template for float only");
    BBCU_HIP_CALL(bbhip_fp32_RealToBinary_Forward(dev_x_buf, dev_y_buf, depth_modulation_size, frame_modulation_size, input_range_lo, input_range_hi,
                                                  point_size, x_depth_size, x_frame_size, x_frame_stride, y_frame_stride, binarize ? 1 : 0, streamId));
    return 0;
}
/* the reference's device kernel takes the bit as value > 0.5 whatever the layer's mode: binarize = 1 */
template <typename T = float>
inline int bbcu_bit_RealToBinary_Forward(T const *dev_x_buf, int *dev_y_buf, unsigned int depth_modulation_size, unsigned int frame_modulation_size,
        T input_range_lo, T input_range_hi, unsigned int point_size, unsigned int x_depth_size, unsigned int x_frame_size,
        unsigned int x_frame_stride, unsigned int y_frame_stride, cudaStream_t streamId = 0)
{
    static_assert(sizeof(T) == sizeof(float), "the reference instantiates this template for float only");
    BBCU_HIP_CALL(bbhip_fp32_bit_RealToBinary_Forward(dev_x_buf, dev_y_buf, depth_modulation_size, frame_modulation_size, input_range_lo,
                                                      input_range_hi, point_size, x_depth_size, x_frame_size, x_frame_stride, y_frame_stride, 1,
                                                      streamId));
    return 0;
}
inline int bbcu_fp32_BinaryToReal_Forward(float const *dev_x_buf, float *dev_y_buf, int node_mux_size, int frame_mux_size, int y_node_size,
        int x_frame_stride, int y_frame_size, int y_frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_BinaryToReal_Forward(dev_x_buf, dev_y_buf, node_mux_size, frame_mux_size, y_node_size, x_frame_stride, y_frame_size,
                                                  y_frame_stride, streamId));
    return 0;
}
inline int bbcu_bit_fp32_BinaryToReal_Forward(int const *dev_x_buf, float *dev_y_buf, int node_mux_size, int frame_mux_size, int y_node_size,
        int x_frame_stride, int y_frame_size, int y_frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_bit_fp32_BinaryToReal_Forward(dev_x_buf, dev_y_buf, node_mux_size, frame_mux_size, y_node_size, x_frame_stride,
                                                      y_frame_size, y_frame_stride, streamId));
    return 0;
}
inline int bbcu_fp32_BinaryToReal_Backward(float const *dev_dy_buf, float *dev_dx_buf, int node_mux_size, int frame_mux_size, int y_node_size,
        int x_frame_stride, int y_frame_size, int y_frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_BinaryToReal_Backward(dev_dy_buf, dev_dx_buf, node_mux_size, frame_mux_size, y_node_size, x_frame_stride,
                                                   y_frame_size, y_frame_stride, streamId));
    return 0;
}

/* ---- Binarize / HardTanh, include/bbcu/bbcu.h:1223-1276 ---- */
inline int bbcu_fp32_Binarize_Forward(const float *dev_x_buf, float *dev_y_buf, float binary_th, float binary_low, float binary_high,
        int node_size, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_Binarize_Forward(dev_x_buf, dev_y_buf, binary_th, binary_low, binary_high, node_size, frame_size, frame_stride, streamId));
    return 0;
}
inline int bbcu_fp32_bit_Binarize_Forward(float const *dev_x_buf, int *dev_y_buf, float binary_th, int node_size, int frame_size,
        int x_frame_stride, int y_frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_bit_Binarize_Forward(dev_x_buf, dev_y_buf, binary_th, node_size, frame_size, x_frame_stride, y_frame_stride, streamId));
    return 0;
}
inline int bbcu_fp32_HardTanh_Forward(float const *dev_x_buf, float *dev_y_buf, float limit_min, float limit_max, int node_size, int frame_size,
        int frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_HardTanh_Forward(dev_x_buf, dev_y_buf, limit_min, limit_max, node_size, frame_size, frame_stride, streamId));
    return 0;
}
inline int bbcu_fp32_HardTanh_Backward(const float *dev_x_buf, const float *dev_dy_buf, float *dev_dx_buf, float limit_min, float limit_max,
        int node_size, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_HardTanh_Backward(dev_x_buf, dev_dy_buf, dev_dx_buf, limit_min, limit_max, node_size, frame_size, frame_stride, streamId));
    return 0;
}

/* ---- MaxPooling / UpSampling, include/bbcu/bbcu.h:949-1068 ---- */
inline int bbcu_fp32_MaxPooling_Forward(float const *dev_x_buf, float *dev_y_buf, int *dev_argmax_buf, int filter_h_size, int filter_w_size,
        int input_w_size, int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size, int frame_stride,
        cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_MaxPooling_Forward(dev_x_buf, dev_y_buf, dev_argmax_buf, filter_h_size, filter_w_size, input_w_size, input_h_size,
                                                output_w_size, output_h_size, c_size, frame_size, frame_stride, streamId));
    return 0;
}
inline int bbcu_bit_MaxPooling_Forward(int const *dev_x_buf, int *dev_y_buf, int filter_h_size, int filter_w_size, int input_w_size,
        int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_bit_MaxPooling_Forward(dev_x_buf, dev_y_buf, filter_h_size, filter_w_size, input_w_size, input_h_size, output_w_size,
                                               output_h_size, c_size, frame_size, frame_stride, streamId));
    return 0;
}
inline int bbcu_fp32_MaxPooling_Backward(int const *dev_argmax_buf, float const *dev_dy_buf, float *dev_dx_buf, int filter_h_size,
        int filter_w_size, int input_w_size, int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size,
        int frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_MaxPooling_Backward(dev_argmax_buf, dev_dy_buf, dev_dx_buf, filter_h_size, filter_w_size, input_w_size, input_h_size,
                                                 output_w_size, output_h_size, c_size, frame_size, frame_stride, streamId));
    return 0;
}
inline int bbcu_bit_fp32_MaxPooling_Backward(int const *dev_x_buf, float const *dev_dy_buf, float *dev_dx_buf, int filter_h_size,
        int filter_w_size, int input_w_size, int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size,
        int forward_frame_stride, int backward_frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_bit_fp32_MaxPooling_Backward(dev_x_buf, dev_dy_buf, dev_dx_buf, filter_h_size, filter_w_size, input_w_size, input_h_size,
                                                     output_w_size, output_h_size, c_size, frame_size, forward_frame_stride,
                                                     backward_frame_stride, streamId));
    return 0;
}
inline int bbcu_fp32_UpSampling_Forward(float const *dev_x_buf, float *dev_y_buf, int input_w_size, int input_h_size, int c_size,
        int filter_w_size, int filter_h_size, int fill, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_UpSampling_Forward(dev_x_buf, dev_y_buf, input_w_size, input_h_size, c_size, filter_w_size, filter_h_size, fill,
                                                frame_size, frame_stride, streamId));
    return 0;
}
inline int bbcu_bit_UpSampling_Forward(int const *dev_x_buf, int *dev_y_buf, int input_w_size, int input_h_size, int c_size,
        int filter_w_size, int filter_h_size, int fill, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_bit_UpSampling_Forward(dev_x_buf, dev_y_buf, input_w_size, input_h_size, c_size, filter_w_size, filter_h_size, fill,
                                               frame_size, frame_stride, streamId));
    return 0;
}
inline int bbcu_fp32_UpSampling_Backward(float const *dev_dy_buf, float *dev_dx_buf, int input_w_size, int input_h_size, int c_size,
        int filter_w_size, int filter_h_size, int fill, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_UpSampling_Backward(dev_dy_buf, dev_dx_buf, input_w_size, input_h_size, c_size, filter_w_size, filter_h_size, fill,
                                                 frame_size, frame_stride, streamId));
    return 0;
}

/* ---- bbcu_Shuffle_Forward<T> / bbcu_Shuffle_Backward<T>, include/bbcu/bbcu.h:1194-1216 (T = int or float: rows of 32-bit words) ---- */
template <typename T>
int bbcu_Shuffle_Forward(T const *dev_x_buf, T *dev_y_buf, unsigned int y_unit_size, unsigned int node_size, unsigned int frame_size,
                         unsigned int frame_stride, cudaStream_t streamId = 0)
{
    static_assert(sizeof(T) == 4, "rows of 32-bit words");
    BBCU_HIP_CALL(bbhip_Shuffle_Forward(reinterpret_cast<int const *>(dev_x_buf), reinterpret_cast<int *>(dev_y_buf), y_unit_size, node_size,
                                        frame_size, frame_stride, streamId));
    return 0;
}
template <typename T>
int bbcu_Shuffle_Backward(T const *dev_dy_buf, T *dev_dx_buf, unsigned int y_unit_size, unsigned int node_size, unsigned int frame_size,
                          unsigned int frame_stride, cudaStream_t streamId = 0)
{
    static_assert(sizeof(T) == 4, "rows of 32-bit words");
    BBCU_HIP_CALL(bbhip_Shuffle_Backward(reinterpret_cast<int const *>(dev_dy_buf), reinterpret_cast<int *>(dev_dx_buf), y_unit_size, node_size,
                                         frame_size, frame_stride, streamId));
    return 0;
}

/* ---- Im2Col / Col2Im, include/bbcu/bbcu.h:1076-1186 ---- */
inline int bbcu_fp32_Im2Col_Forward(float const *dev_x_buf, float *dev_y_buf, int x_stride, int y_stride, int x_offset, int y_offset,
        int input_frame_size, int input_frame_stride, int input_w_size, int input_h_size, int input_c_size, int output_w_size,
        int output_h_size, int output_frame_stride, int filter_w_size, int filter_h_size, int border_mode, float border_value,
        cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_Im2Col_Forward(dev_x_buf, dev_y_buf, x_stride, y_stride, x_offset, y_offset, input_frame_size, input_frame_stride,
            input_w_size, input_h_size, input_c_size, output_w_size, output_h_size, output_frame_stride, filter_w_size, filter_h_size,
            border_mode, border_value, streamId));
    return 0;
}
inline int bbcu_bit_Im2Col_Forward(int const *dev_x_buf, int *dev_y_buf, int x_stride, int y_stride, int x_offset, int y_offset,
        int input_frame_size, int input_frame_stride, int input_w_size, int input_h_size, int input_c_size, int output_w_size,
        int output_h_size, int output_frame_stride, int filter_w_size, int filter_h_size, int border_mode, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_bit_Im2Col_Forward(dev_x_buf, dev_y_buf, x_stride, y_stride, x_offset, y_offset, input_frame_size, input_frame_stride,
            input_w_size, input_h_size, input_c_size, output_w_size, output_h_size, output_frame_stride, filter_w_size, filter_h_size,
            border_mode, streamId));
    return 0;
}
inline int bbcu_fp32_Im2Col_Backward(float const *dev_fy_buf, float *dev_dx_buf, int x_stride, int y_stride, int x_offset, int y_offset,
        int input_frame_size, int input_frame_stride, int input_w_size, int input_h_size, int input_c_size, int output_w_size,
        int output_h_size, int output_frame_stride, int filter_w_size, int filter_h_size, cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_Im2Col_Backward(dev_fy_buf, dev_dx_buf, x_stride, y_stride, x_offset, y_offset, input_frame_size,
            input_frame_stride, input_w_size, input_h_size, input_c_size, output_w_size, output_h_size, output_frame_stride, filter_w_size,
            filter_h_size, streamId));
    return 0;
}
inline int bbcu_fp32_Col2Im_Forward(float const *dev_x_buf, float *dev_y_buf, int w_size, int h_size, int c_size, int input_frame_stride,
        int output_frame_size, int output_frame_stride, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_fp32_Col2Im_Forward(dev_x_buf, dev_y_buf, w_size, h_size, c_size, input_frame_stride, output_frame_size, output_frame_stride, streamId)); return 0; }
inline int bbcu_bit_Col2Im_Forward(int const *dev_x_buf, int *dev_y_buf, int w_size, int h_size, int c_size, int input_frame_stride,
        int output_frame_size, int output_frame_stride, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_bit_Col2Im_Forward(dev_x_buf, dev_y_buf, w_size, h_size, c_size, input_frame_stride, output_frame_size, output_frame_stride, streamId)); return 0; }
inline int bbcu_fp32_Col2Im_Backward(float const *dev_dy_buf, float *dev_dx_buf, int w_size, int h_size, int c_size, int input_frame_stride,
        int output_frame_size, int output_frame_stride, cudaStream_t streamId = 0)
{ BBCU_HIP_CALL(bbhip_fp32_Col2Im_Backward(dev_dy_buf, dev_dx_buf, w_size, h_size, c_size, input_frame_stride, output_frame_size, output_frame_stride, streamId)); return 0; }

/* ---- bbcu_LossSoftmaxCrossEntropy<T>, include/bbcu/bbcu.h:1506-1519; bbcu_MetricsCategoricalAccuracy<T>, :1540-1553 (T = float) ---- */
template <typename T>
int bbcu_LossSoftmaxCrossEntropy(T const *dev_y_buf, T const *dev_t_buf, T *dev_dy_buf, double *dev_loss_buf, T t_sum, int pix_size,
                                 int ch_size, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    static_assert(std::is_same<T, float>::value, "fp32 frames");
    BBCU_HIP_CALL(bbhip_fp32_LossSoftmaxCrossEntropy(dev_y_buf, dev_t_buf, dev_dy_buf, dev_loss_buf, t_sum, pix_size, ch_size, frame_size,
                                                     frame_stride, streamId));
    return 0;
}
template <typename T>
int bbcu_MetricsCategoricalAccuracy(T const *dev_y_buf, T const *dev_t_buf, int *dev_accuracy_buf, int *dev_category_buf, int pix_size,
                                    int ch_size, int frame_size, int frame_stride, cudaStream_t streamId = 0)
{
    static_assert(std::is_same<T, float>::value, "fp32 frames");
    BBCU_HIP_CALL(bbhip_fp32_MetricsCategoricalAccuracy(dev_y_buf, dev_t_buf, dev_accuracy_buf, dev_category_buf, pix_size, ch_size, frame_size,
                                                        frame_stride, streamId));
    return 0;
}

/* ---- bbcu_fp32_OptimizerAdam, include/bbcu/bbcu.h:1560-1572 ---- */
inline int bbcu_fp32_OptimizerAdam(int size, int const *dev_size_table, float *const *dev_params_buf_table, float *const *dev_grads_buf_table,
                                   float *const *dev_m_buf_table, float *const *dev_v_buf_table, float lr_t, float beta1, float beta2,
                                   cudaStream_t streamId = 0)
{
    BBCU_HIP_CALL(bbhip_fp32_OptimizerAdam(size, dev_size_table, dev_params_buf_table, dev_grads_buf_table, dev_m_buf_table, dev_v_buf_table,
                                           lr_t, beta1, beta2, streamId));
    return 0;
}

#endif  /* BBCU_HIP_BINDING_H_ */
