"""ctypes binding of the C ABI in include/bbhip.h.  Device memory and streams come from torch; nothing here computes."""
import ctypes as C
import os

from .build import LIB_PATH

_lib = None

_vp, _i, _f, _u = C.c_void_p, C.c_int, C.c_float, C.c_uint

_SIGNATURES = {
    "bbhip_GetDeviceCount": (C.c_int, []),
    "bbhip_GetDevice": (C.c_int, []),
    "bbhip_SetDevice": (None, [_i]),
    "bbhip_SetHostOnly": (None, [_i]),
    "bbhip_IsHostOnly": (C.c_int, []),
    "bbhip_IsDeviceAvailable": (C.c_int, []),
    "bbhip_GetLastErrorString": (C.c_char_p, []),
    "bbhip_LocalHeap_Malloc": (C.c_void_p, [C.c_size_t]),
    "bbhip_LocalHeap_Free": (None, [_vp]),
    "bbhip_LocalHeap_GetMaxAllocSize": (C.c_size_t, []),
    "bbhip_LocalHeap_GetAllocatedSize": (C.c_size_t, []),
    "bbhip_LocalHeap_GarbageCollect": (None, []),
    "bbhip_Malloc": (C.c_int, [C.POINTER(C.c_void_p), C.c_size_t]),
    "bbhip_Free": (C.c_int, [_vp]),
    "bbhip_MallocHost": (C.c_int, [C.POINTER(C.c_void_p), C.c_size_t]),
    "bbhip_FreeHost": (C.c_int, [_vp]),
    "bbhip_Memcpy": (C.c_int, [_vp, _vp, C.c_size_t, _i]),
    "bbhip_Memset": (C.c_int, [_vp, _i, C.c_size_t]),
    "bbhip_DeviceSynchronize": (C.c_int, []),
    "bbhip_KernelTimer_Enable": (None, [_i]),
    "bbhip_KernelTimer_Read": (C.c_int, [_i, C.POINTER(C.c_float), C.POINTER(C.c_int)]),
    "bbhip_ReserveScratch": (C.c_int, [C.c_size_t]),
    "bbhip_ReleaseScratch": (C.c_int, []),
    "bbhip_GetScratchSize": (C.c_size_t, []),
    "bbhip_GetSwitch": (C.c_int, [C.c_char_p]),
    "bbhip_SetDxMode": (None, [_i]),
    "bbhip_HintInputNodeSize": (None, [_i]),
    "bbhip_PackedRowWords": (C.c_int, [_i]),
    "bbhip_HintPackedInput": (None, [_vp, _i, _i, _i]),
    "bbhip_HintPackedOutput": (None, [_vp, _i, _i]),
    "bbhip_HintTableGradientOverwrite": (None, [_i]),
    "bbhip_HintPreparedTables": (None, [_vp, C.c_size_t, _i]),
    "bbhip_PreparedTablesBytes": (C.c_size_t, [_i, _i]),
    "bbhip_GetDxMode": (C.c_int, []),
    "bbhip_fp32_Vector_set": (C.c_int, [_vp, _f, _i, _vp]),
    "bbhip_fp32_Vector_clamp": (C.c_int, [_vp, _vp, _f, _f, _i, _vp]),
    "bbhip_fp32_Vector_add_ex": (C.c_int, [_vp, _vp, _vp, _f, _f, _f, _i, _vp]),
    "bbhip_fp32_Vector_mul_ex": (C.c_int, [_vp, _vp, _vp, _f, _f, _i, _vp]),
    "bbhip_fp32_Vector_div_ex": (C.c_int, [_vp, _vp, _vp, _f, _f, _f, _f, _i, _vp]),
    "bbhip_fp32_Vector_sqrt": (C.c_int, [_vp, _vp, _i, _vp]),
    "bbhip_fp32_Vector_exp": (C.c_int, [_vp, _vp, _i, _vp]),
    "bbhip_fp32_Vector_min": (C.c_int, [_vp, _vp, _vp, _i, _vp]),
    "bbhip_fp32_Vector_min_v": (C.c_int, [_vp, _vp, _f, _i, _vp]),
    "bbhip_fp32_Vector_max": (C.c_int, [_vp, _vp, _vp, _i, _vp]),
    "bbhip_fp32_Vector_max_v": (C.c_int, [_vp, _vp, _f, _i, _vp]),
    "bbhip_fp32_OptimizerAdam": (C.c_int, [_i, _vp, _vp, _vp, _vp, _vp, _f, _f, _f, _vp]),
    "bbhip_fp32_OptimizerAdam_Update": (C.c_int, [_i, _vp, _vp, _vp, _vp, _vp, _f, _f, _f, _vp]),
    "bbhip_fp32_Im2Col_Forward": (C.c_int, [_vp, _vp] + [_i] * 15 + [_f, _vp]),
    "bbhip_bit_Im2Col_Forward": (C.c_int, [_vp, _vp] + [_i] * 15 + [_vp]),
    "bbhip_fp32_Im2Col_Backward": (C.c_int, [_vp, _vp] + [_i] * 14 + [_vp]),
    "bbhip_fp32_Col2Im_Forward": (C.c_int, [_vp, _vp] + [_i] * 6 + [_vp]),
    "bbhip_bit_Col2Im_Forward": (C.c_int, [_vp, _vp] + [_i] * 6 + [_vp]),
    "bbhip_fp32_Col2Im_Backward": (C.c_int, [_vp, _vp] + [_i] * 6 + [_vp]),
    "bbhip_fp32_StochasticMaxPooling2x2_Forward": (C.c_int, [_vp, _vp] + [_i] * 7 + [_vp]),
    "bbhip_fp32_StochasticMaxPooling2x2_Backward": (C.c_int, [_vp, _vp, _vp] + [_i] * 7 + [_vp]),
    "bbhip_fp32_AverageLut_Forward": (C.c_int, [_vp, _vp, _vp] + [_i] * 6 + [_vp]),
    "bbhip_fp32_AverageLut_ForwardSum": (C.c_int, [_vp, _vp, _vp] + [_i] * 6 + [_vp]),
    "bbhip_bit_AverageLut_Forward": (C.c_int, [_vp, _vp, _vp] + [_i] * 4 + [_vp]),
    "bbhip_fp32_AverageLut_Backward": (C.c_int, [_vp, _vp, _vp] + [_i] * 5 + [_vp]),
    "bbhip_fp32_ClassifierTail_ForwardBackward": (C.c_int, [_vp] * 9 + [_f] + [_i] * 7 + [_vp]),
    "bbhip_fp32_MaxLut_Forward": (C.c_int, [_vp, _vp, _vp] + [_i] * 6 + [_vp]),
    "bbhip_bit_MaxLut_Forward": (C.c_int, [_vp, _vp, _vp] + [_i] * 4 + [_vp]),
    "bbhip_fp32_MaxLut_Backward": (C.c_int, [_vp, _vp, _vp, _vp] + [_i] * 6 + [_vp]),
    "bbhip_bit_fp32_MaxLut_Backward": (C.c_int, [_vp, _vp, _vp, _vp] + [_i] * 6 + [_vp]),
    "bbhip_fp32_Reduce_Forward": (C.c_int, [_vp, _vp] + [_i] * 4 + [_vp]),
    "bbhip_bit_fp32_Reduce_Forward": (C.c_int, [_vp, _vp] + [_i] * 5 + [_vp]),
    "bbhip_fp32_Reduce_Backward": (C.c_int, [_vp, _vp] + [_i] * 4 + [_vp]),
    "bbhip_fp32_LossMeanSquaredError": (C.c_int, [_vp, _vp, _vp, _vp] + [_i] * 4 + [_f, C.c_double, _vp]),
    "bbhip_fp32_MetricsMeanSquaredError": (C.c_int, [_vp, _vp, _vp] + [_i] * 4 + [_vp]),
    "bbhip_fp32_LossSoftmaxCrossEntropy": (C.c_int, [_vp, _vp, _vp, _vp, _f] + [_i] * 4 + [_vp]),
    "bbhip_fp32_MetricsCategoricalAccuracy": (C.c_int, [_vp, _vp, _vp, _vp] + [_i] * 4 + [_vp]),
    "bbhip_fp32_StochasticBatchNormalization_ForwardTraining": (C.c_int, [_vp] * 6 + [_f, _f, _f, _i, _i, _i, _vp]),
    "bbhip_fp32_StochasticBatchNormalization_ReForward": (C.c_int, [_vp] * 4 + [_f, _f, _i, _i, _i, _vp]),
    "bbhip_fp32_StochasticBatchNormalization_ForwardInference": (C.c_int, [_vp] * 4 + [_f, _f, _i, _i, _i, _vp]),
    "bbhip_fp32_StochasticBatchNormalization_Backward": (C.c_int, [_vp] * 5 + [_f, _f, _i, _i, _i, _i, _vp]),
    "bbhip_fp32_RealToBinary_Forward": (C.c_int, [_vp, _vp, _u, _u, _f, _f] + [_u] * 5 + [_i, _vp]),
    "bbhip_fp32_bit_RealToBinary_Forward": (C.c_int, [_vp, _vp, _u, _u, _f, _f] + [_u] * 5 + [_i, _vp]),
    "bbhip_fp32_BinaryToReal_Forward": (C.c_int, [_vp, _vp] + [_i] * 6 + [_vp]),
    "bbhip_bit_fp32_BinaryToReal_Forward": (C.c_int, [_vp, _vp] + [_i] * 6 + [_vp]),
    "bbhip_fp32_BinaryToReal_Backward": (C.c_int, [_vp, _vp] + [_i] * 6 + [_vp]),
    "bbhip_fp32_Binarize_Forward": (C.c_int, [_vp, _vp, _f, _f, _f, _i, _i, _i, _vp]),
    "bbhip_fp32_bit_Binarize_Forward": (C.c_int, [_vp, _vp, _f, _i, _i, _i, _i, _vp]),
    "bbhip_fp32_HardTanh_Forward": (C.c_int, [_vp, _vp, _f, _f, _i, _i, _i, _vp]),
    "bbhip_fp32_HardTanh_Backward": (C.c_int, [_vp, _vp, _vp, _f, _f, _i, _i, _i, _vp]),
    "bbhip_fp32_MaxPooling_Forward": (C.c_int, [_vp, _vp, _vp] + [_i] * 9 + [_vp]),
    "bbhip_bit_MaxPooling_Forward": (C.c_int, [_vp, _vp] + [_i] * 9 + [_vp]),
    "bbhip_fp32_MaxPooling_Backward": (C.c_int, [_vp, _vp, _vp] + [_i] * 9 + [_vp]),
    "bbhip_bit_fp32_MaxPooling_Backward": (C.c_int, [_vp, _vp, _vp] + [_i] * 10 + [_vp]),
    "bbhip_fp32_UpSampling_Forward": (C.c_int, [_vp, _vp] + [_i] * 8 + [_vp]),
    "bbhip_bit_UpSampling_Forward": (C.c_int, [_vp, _vp] + [_i] * 8 + [_vp]),
    "bbhip_fp32_UpSampling_Backward": (C.c_int, [_vp, _vp] + [_i] * 8 + [_vp]),
    "bbhip_Shuffle_Forward": (C.c_int, [_vp, _vp] + [_u] * 4 + [_vp]),
    "bbhip_Shuffle_Backward": (C.c_int, [_vp, _vp] + [_u] * 4 + [_vp]),
    "bbhip_fp32_ConvBitToReal": (C.c_int, [_vp, _vp, _f, _f, _i, _i, _i, _i, _vp]),
    "bbhip_fp32_StochasticLut_Forward": (C.c_int, [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _vp]),
    "bbhip_fp32_StochasticLut_Forward_NoAlloc": (C.c_int, [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _vp]),
    "bbhip_fp32_StochasticLut_ForwardClampW": (C.c_int, [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _f, _f, _vp]),
    "bbhip_bit_fp32_StochasticLut_Forward": (C.c_int, [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _vp]),
    "bbhip_bit_bit_fp32_StochasticLut_Forward": (C.c_int, [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f, _vp]),
    "bbhip_fp32_StochasticLut_Backward": (C.c_int, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp] + [_i] * 9 + [_f, _vp]),
    "bbhip_bit_fp32_StochasticLut_Backward": (C.c_int, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp] + [_i] * 9 + [_f, _vp]),
    "bbhip_fp32_DifferentiableLutN_ForwardTraining": (C.c_int, [_i] + [_vp] * 8 + [_f] * 4 + [_i] * 5 + [_vp]),
    "bbhip_bit_fp32_DifferentiableLutN_ForwardTraining": (C.c_int, [_i] + [_vp] * 8 + [_f] * 4 + [_i] * 4 + [_vp]),
    "bbhip_fp32_DifferentiableLutN_ForwardTrainingClampW": (C.c_int, [_i] + [_vp] * 8 + [_f] * 4 + [_i] * 5 + [_f, _f, _vp]),
    "bbhip_bit_fp32_DifferentiableLutN_ForwardTrainingClampW": (C.c_int, [_i] + [_vp] * 8 + [_f] * 4 + [_i] * 4 + [_f, _f, _vp]),
    "bbhip_fp32_DifferentiableLutN_ForwardInference": (C.c_int, [_i] + [_vp] * 6 + [_f] * 3 + [_i] * 5 + [_vp]),
    "bbhip_bit_fp32_DifferentiableLutN_ForwardInference": (C.c_int, [_i] + [_vp] * 6 + [_f] * 3 + [_i] * 4 + [_vp]),
    "bbhip_fp32_DifferentiableLutN_Backward": (C.c_int, [_i] + [_vp] * 12 + [_f] * 3 + [_i] * 9 + [_vp]),
    "bbhip_bit_fp32_DifferentiableLutN_Backward": (C.c_int, [_i] + [_vp] * 12 + [_f] * 3 + [_i] * 9 + [_vp]),
    "bbhip_fp32_DifferentiableLutN_ForwardNoBn": (C.c_int, [_i] + [_vp] * 4 + [_f] + [_i] * 5 + [_vp]),
    "bbhip_bit_BinaryLut6_Forward": (C.c_int, [_vp] * 4 + [_i] * 3 + [_vp]),
    "bbhip_bit_BinaryLutN_Forward": (C.c_int, [_i] + [_vp] * 4 + [_i] * 3 + [_vp]),
}


class BbhipError(RuntimeError):
    pass


def lib():
    """The loaded library. Fails loudly when it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise BbhipError("%s is missing: build it with `python -m binarybrain_amd.build` "
                             "(or __graft_entry__.build())" % LIB_PATH)
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def exported_symbols():
    return sorted(_SIGNATURES)


def check(rc):
    if rc != 0:
        raise BbhipError(lib().bbhip_GetLastErrorString().decode())


def ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def stream_ptr():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)
