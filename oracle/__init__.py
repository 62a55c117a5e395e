"""TEST INFRASTRUCTURE — ctypes access to the CPU oracle.

Two libraries sit behind this module:

* ``liboracle.so``      — the plain-C restatement of the reference's CPU algorithm (``bb_oracle.c``).
* ``_ref/libbbref.so``  — the reference's own CPU headers compiled behind ``ref_shim.cpp`` (present only where it
  was built from the reference tree).

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this module; the
shipped package never does.  Arrays are numpy, node-major / frame-minor, C-contiguous: fp32 buffers are
``[nodes, stride]`` float32, bit buffers ``[nodes, stride_words]`` int32 with frame f at word f>>5, bit f&31.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_SO = os.path.join(_HERE, "liboracle.so")
_REF_SO = os.path.join(_HERE, "_ref", "libbbref.so")

_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")


def build(force=False):
    """Compile liboracle.so (and _ref/libbbref.so where the reference tree is present)."""
    if force or not os.path.exists(_ORACLE_SO):
        subprocess.check_call(["make", "-C", _HERE, "liboracle.so"] + (["-B"] if force else []))
    if os.path.isdir("/root/reference/include/bb") and (force or not os.path.exists(_REF_SO)):
        subprocess.check_call(["make", "-C", _HERE, "ref"])


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_ORACLE_SO):
            build()
        _lib = C.CDLL(_ORACLE_SO)
    return _lib


def have_ref():
    return os.path.exists(_REF_SO)


def ref():
    global _ref
    if _ref is None:
        _ref = C.CDLL(_REF_SO)
    return _ref


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


# ----------------------------------------------------------------------------------------------
#  restatement (liboracle.so)
# ----------------------------------------------------------------------------------------------

def vector_clamp(src, lo=0.0, hi=1.0):
    src = _c(src, np.float32)
    dst = np.empty_like(src)
    lib().oracle_fp32_Vector_clamp(_ptr(dst), _ptr(src), C.c_float(lo), C.c_float(hi), C.c_int(src.size))
    return dst


_VEC_OPS = {"add_ex": 0, "mul_ex": 1, "div_ex": 2, "sqrt": 3, "exp": 4, "min": 5, "min_v": 6, "max": 7, "max_v": 8}


def vector_op(name, src0, src1=None, a=0.0, b=0.0, c=0.0, d=0.0):
    """Elementwise fp32 vector operation ``name`` of the reference's Tensor arithmetic."""
    src0 = _c(src0, np.float32)
    src1 = None if src1 is None else _c(src1, np.float32)
    dst = np.empty_like(src0)
    lib().oracle_fp32_Vector_op(C.c_int(_VEC_OPS[name]), _ptr(dst), _ptr(src0), _ptr(src1), C.c_float(a), C.c_float(b),
                                C.c_float(c), C.c_float(d), C.c_int(src0.size))
    return dst


def adam_lr_t(learning_rate, b1, b2):
    """Bias-corrected rate in fp32, as include/bb/OptimizerAdam.h:171 computes it."""
    one = np.float32(1.0)
    return np.float32(np.float32(np.float32(learning_rate) * np.sqrt(one - np.float32(b2), dtype=np.float32)) / (one - np.float32(b1)))


def adam_steps(param, grads, learning_rate=0.001, beta1=0.9, beta2=0.999):
    """Run len(grads) Adam updates on one tensor; returns (param, m, v) after the last step."""
    p = _c(param, np.float32).copy()
    m = np.zeros_like(p); v = np.zeros_like(p)
    b1 = np.float32(beta1); b2 = np.float32(beta2)
    for g in grads:
        g = _c(g, np.float32)
        lib().oracle_fp32_OptimizerAdam(C.c_int(p.size), _ptr(p), _ptr(g), _ptr(m), _ptr(v), C.c_float(adam_lr_t(learning_rate, b1, b2)),
                                        C.c_float(beta1), C.c_float(beta2))
        b1 = np.float32(b1 * np.float32(beta1)); b2 = np.float32(b2 * np.float32(beta2))
    return p, m, v


BORDER_MODES = {"constant": 0, "reflect": 1, "reflect_101": 2, "replicate": 3, "wrap": 4}


def im2col_geometry(h, w, fh, fw, ys=1, xs=1, padding="valid"):
    """(oh, ow, y_offset, x_offset) as include/bb/ConvolutionIm2Col.h:183-198 computes them."""
    if padding == "valid":
        return ((h - fh + 1) + (ys - 1)) // ys, ((w - fw + 1) + (xs - 1)) // xs, 0, 0
    assert padding == "same"
    return (h + ys - 1) // ys, (w + xs - 1) // xs, (fh - 1) // 2, (fw - 1) // 2


def im2col_forward(x, c, h, w, frames, fh, fw, ys=1, xs=1, padding="valid", border="reflect_101", border_value=0.0, bit=False):
    """x: [c*h*w, stride] fp32 (or packed int32 words when bit) -> y: [c*fh*fw, stride'] over frames*oh*ow frames."""
    oh, ow, yo, xo = im2col_geometry(h, w, fh, fw, ys, xs, padding)
    of = frames * oh * ow
    if bit:
        x = _c(x, np.int32)
        y = np.zeros((c * fh * fw, (of + 31) // 32), np.int32)
        lib().oracle_bit_Im2Col_Forward(_ptr(x), _ptr(y), C.c_int(xs), C.c_int(ys), C.c_int(xo), C.c_int(yo), C.c_int(frames),
                                        C.c_int(x.shape[1]), C.c_int(w), C.c_int(h), C.c_int(c), C.c_int(ow), C.c_int(oh),
                                        C.c_int(y.shape[1]), C.c_int(fw), C.c_int(fh), C.c_int(BORDER_MODES[border]))
    else:
        x = _c(x, np.float32)
        y = np.zeros((c * fh * fw, of), np.float32)
        lib().oracle_fp32_Im2Col_Forward(_ptr(x), _ptr(y), C.c_int(xs), C.c_int(ys), C.c_int(xo), C.c_int(yo), C.c_int(frames),
                                         C.c_int(x.shape[1]), C.c_int(w), C.c_int(h), C.c_int(c), C.c_int(ow), C.c_int(oh),
                                         C.c_int(y.shape[1]), C.c_int(fw), C.c_int(fh), C.c_int(BORDER_MODES[border]),
                                         C.c_float(border_value))
    return y


def im2col_backward(dy, c, h, w, frames, fh, fw, ys=1, xs=1, padding="valid"):
    oh, ow, yo, xo = im2col_geometry(h, w, fh, fw, ys, xs, padding)
    dy = _c(dy, np.float32)
    dx = np.zeros((c * h * w, frames), np.float32)
    lib().oracle_fp32_Im2Col_Backward(_ptr(dy), _ptr(dx), C.c_int(xs), C.c_int(ys), C.c_int(xo), C.c_int(yo), C.c_int(frames),
                                      C.c_int(frames), C.c_int(w), C.c_int(h), C.c_int(c), C.c_int(ow), C.c_int(oh),
                                      C.c_int(dy.shape[1]), C.c_int(fw), C.c_int(fh))
    return dx


def col2im_forward(x, c, h, w, frames, bit=False):
    """x: [c, frames*h*w] -> y: [c*h*w, frames]"""
    if bit:
        x = _c(x, np.int32)
        y = np.zeros((c * h * w, (frames + 31) // 32), np.int32)
        lib().oracle_bit_Col2Im_Forward(_ptr(x), _ptr(y), C.c_int(w), C.c_int(h), C.c_int(c), C.c_int(x.shape[1]), C.c_int(frames), C.c_int(y.shape[1]))
    else:
        x = _c(x, np.float32)
        y = np.zeros((c * h * w, frames), np.float32)
        lib().oracle_fp32_Col2Im_Forward(_ptr(x), _ptr(y), C.c_int(w), C.c_int(h), C.c_int(c), C.c_int(x.shape[1]), C.c_int(frames), C.c_int(frames))
    return y


def col2im_backward(dy, c, h, w, frames):
    dy = _c(dy, np.float32)
    dx = np.zeros((c, frames * h * w), np.float32)
    lib().oracle_fp32_Col2Im_Backward(_ptr(dy), _ptr(dx), C.c_int(w), C.c_int(h), C.c_int(c), C.c_int(dx.shape[1]), C.c_int(frames), C.c_int(dy.shape[1]))
    return dx


def stochastic_maxpool2x2_forward(x, c, h, w, frames):
    x = _c(x, np.float32)
    oh, ow = (h + 1) // 2, (w + 1) // 2
    y = np.zeros((c * oh * ow, x.shape[1]), np.float32)
    lib().oracle_fp32_StochasticMaxPooling2x2_Forward(_ptr(x), _ptr(y), C.c_int(w), C.c_int(h), C.c_int(ow), C.c_int(oh), C.c_int(c),
                                                      C.c_int(frames), C.c_int(x.shape[1]))
    return y


def stochastic_maxpool2x2_backward(x, dy, c, h, w, frames):
    x = _c(x, np.float32); dy = _c(dy, np.float32)
    oh, ow = (h + 1) // 2, (w + 1) // 2
    dx = np.zeros_like(x)
    lib().oracle_fp32_StochasticMaxPooling2x2_Backward(_ptr(x), _ptr(dy), _ptr(dx), C.c_int(w), C.c_int(h), C.c_int(ow), C.c_int(oh),
                                                       C.c_int(c), C.c_int(frames), C.c_int(x.shape[1]))
    return dx


def stochastic_bn_forward_training(x, running_mean, running_var, gamma, beta, momentum, frame_size):
    """Per-node batch normalisation with scalar gamma / beta, training pass (the reference's generic host loop,
    include/bb/StochasticBatchNormalization.h:535-597) -> (y, mean, rstd, running_mean', running_var')."""
    x = _c(x, np.float32)
    y = np.zeros_like(x)
    nodes = x.shape[0]
    mean = np.zeros(nodes, np.float32); rstd = np.zeros(nodes, np.float32)
    rm = _c(running_mean, np.float32).copy(); rv = _c(running_var, np.float32).copy()
    lib().oracle_fp32_StochasticBatchNormalization_ForwardTraining(_ptr(x), _ptr(y), _ptr(mean), _ptr(rstd), _ptr(rm), _ptr(rv),
                                                                   C.c_float(gamma), C.c_float(beta), C.c_float(momentum), C.c_int(nodes),
                                                                   C.c_int(frame_size), C.c_int(x.shape[1]))
    return y, mean, rstd, rm, rv


def stochastic_bn_reforward(x, mean, rstd, gamma, beta, frame_size):
    x = _c(x, np.float32); mean = _c(mean, np.float32); rstd = _c(rstd, np.float32)
    y = np.zeros_like(x)
    lib().oracle_fp32_StochasticBatchNormalization_ReForward(_ptr(x), _ptr(y), _ptr(mean), _ptr(rstd), C.c_float(gamma), C.c_float(beta),
                                                             C.c_int(x.shape[0]), C.c_int(frame_size), C.c_int(x.shape[1]))
    return y


def stochastic_bn_forward_inference(x, running_mean, running_var, gamma, beta, frame_size):
    x = _c(x, np.float32); rm = _c(running_mean, np.float32); rv = _c(running_var, np.float32)
    y = np.zeros_like(x)
    lib().oracle_fp32_StochasticBatchNormalization_ForwardInference(_ptr(x), _ptr(y), _ptr(rm), _ptr(rv), C.c_float(gamma), C.c_float(beta),
                                                                    C.c_int(x.shape[0]), C.c_int(frame_size), C.c_int(x.shape[1]))
    return y


def stochastic_bn_backward(x, dy, mean, rstd, gamma, frame_size):
    x = _c(x, np.float32); dy = _c(dy, np.float32); mean = _c(mean, np.float32); rstd = _c(rstd, np.float32)
    dx = np.zeros_like(dy)
    lib().oracle_fp32_StochasticBatchNormalization_Backward(_ptr(x), _ptr(dy), _ptr(dx), _ptr(mean), _ptr(rstd), C.c_float(gamma),
                                                            C.c_int(dy.shape[0]), C.c_int(frame_size), C.c_int(dy.shape[1]),
                                                            C.c_int(x.shape[1]))
    return dx


def average_lut_forward(x, idx, frame_size, binarize_input=False, binarize_output=True, mean=False):
    """fp32 x [I, stride] -> y [O, stride]: sum (or its sign) of the n wired inputs, the reference's host loop
    (include/bb/AverageLut.h:331-343).  mean: the convention of the reference's CUDA kernel instead, which writes an
    un-binarized output as sum * reciprocal_n with reciprocal_n = (float)1.0 / (float)n (cuda/AverageLut.cu:46-54, 93) —
    the same sum, one fp32 reciprocal, one fp32 product; pinned by its closed form (exactly sum / n when n is a power of two)."""
    x = _c(x, np.float32); idx = _c(idx, np.int32)
    O, n = idx.shape
    y = np.zeros((O, x.shape[1]), np.float32)
    lib().oracle_fp32_AverageLut_Forward(_ptr(x), _ptr(y), _ptr(idx), C.c_int(n), C.c_int(O), C.c_int(frame_size), C.c_int(x.shape[1]),
                                         C.c_int(int(binarize_input)), C.c_int(int(binarize_output)))
    if mean and not binarize_output:
        y = (y * (np.float32(1.0) / np.float32(n))).astype(np.float32)
    return y


def bit_average_lut_forward(xbits, idx, frame_size):
    """packed x [I, words] -> packed y [O, words]: strict majority of the n wired inputs."""
    xbits = _c(xbits, np.int32); idx = _c(idx, np.int32)
    O, n = idx.shape
    y = np.zeros((O, xbits.shape[1]), np.int32)
    lib().oracle_bit_AverageLut_Forward(_ptr(xbits), _ptr(y), _ptr(idx), C.c_int(n), C.c_int(O), C.c_int(frame_size), C.c_int(xbits.shape[1]))
    return y


def average_lut_backward(dy, idx, input_node_size, frame_size):
    dy = _c(dy, np.float32); idx = _c(idx, np.int32)
    O, n = idx.shape
    dx = np.zeros((input_node_size, dy.shape[1]), np.float32)
    lib().oracle_fp32_AverageLut_Backward(_ptr(dy), _ptr(dx), _ptr(idx), C.c_int(n), C.c_int(input_node_size), C.c_int(O),
                                          C.c_int(frame_size), C.c_int(dy.shape[1]))
    return dx


def max_lut_forward(x, idx, frame_size, binarize_input=False, binarize_output=True):
    """fp32 x [I, stride] -> y [O, stride]: the largest of the n wired inputs, not below -1 (or its sign), the reference's host loop
    (include/bb/MaxLut.h:293-318)."""
    x = _c(x, np.float32); idx = _c(idx, np.int32)
    O, n = idx.shape
    y = np.zeros((O, x.shape[1]), np.float32)
    lib().oracle_fp32_MaxLut_Forward(_ptr(x), _ptr(y), _ptr(idx), C.c_int(n), C.c_int(O), C.c_int(frame_size), C.c_int(x.shape[1]),
                                     C.c_int(int(binarize_input)), C.c_int(int(binarize_output)))
    return y


def bit_max_lut_forward(xbits, idx, frame_size):
    """packed x [I, words] -> packed y [O, words]: the OR of the n wired inputs."""
    xbits = _c(xbits, np.int32); idx = _c(idx, np.int32)
    O, n = idx.shape
    y = np.zeros((O, xbits.shape[1]), np.int32)
    lib().oracle_bit_MaxLut_Forward(_ptr(xbits), _ptr(y), _ptr(idx), C.c_int(n), C.c_int(O), C.c_int(frame_size), C.c_int(xbits.shape[1]))
    return y


def max_lut_backward(x, dy, idx, frame_size, binarize_input=False):
    """dx [I, stride]: each node's dy goes to its first largest input (include/bb/MaxLut.h:394-424)."""
    x = _c(x, np.float32); dy = _c(dy, np.float32); idx = _c(idx, np.int32)
    O, n = idx.shape
    dx = np.zeros((x.shape[0], dy.shape[1]), np.float32)
    assert x.shape[1] == dy.shape[1]
    lib().oracle_fp32_MaxLut_Backward(_ptr(x), _ptr(dy), _ptr(dx), _ptr(idx), C.c_int(n), C.c_int(x.shape[0]), C.c_int(O),
                                      C.c_int(frame_size), C.c_int(dy.shape[1]), C.c_int(int(binarize_input)))
    return dx


def bit_max_lut_backward(xbits, dy, idx, frame_size):
    xbits = _c(xbits, np.int32); dy = _c(dy, np.float32); idx = _c(idx, np.int32)
    O, n = idx.shape
    dx = np.zeros((xbits.shape[0], dy.shape[1]), np.float32)
    lib().oracle_bit_MaxLut_Backward(_ptr(xbits), _ptr(dy), _ptr(dx), _ptr(idx), C.c_int(n), C.c_int(xbits.shape[0]), C.c_int(O),
                                     C.c_int(frame_size), C.c_int(xbits.shape[1]), C.c_int(dy.shape[1]))
    return dx


def reduce_forward(x, output_node_size, frame_size):
    """fp32 x [I, stride] -> y [O, stride]: node o is the mean of the inputs o, O + o, 2 O + o, ... (include/bb/Reduce.h:172-190)."""
    x = _c(x, np.float32)
    y = np.zeros((output_node_size, x.shape[1]), np.float32)
    lib().oracle_fp32_Reduce_Forward(_ptr(x), _ptr(y), C.c_int(x.shape[0]), C.c_int(output_node_size), C.c_int(frame_size), C.c_int(x.shape[1]))
    return y


def bit_reduce_forward(xbits, output_node_size, frame_size, y_stride):
    xbits = _c(xbits, np.int32)
    y = np.zeros((output_node_size, y_stride), np.float32)
    lib().oracle_bit_fp32_Reduce_Forward(_ptr(xbits), _ptr(y), C.c_int(xbits.shape[0]), C.c_int(output_node_size), C.c_int(frame_size),
                                         C.c_int(xbits.shape[1]), C.c_int(y_stride))
    return y


def reduce_backward(dy, input_node_size, frame_size):
    dy = _c(dy, np.float32)
    dx = np.zeros((input_node_size, dy.shape[1]), np.float32)
    lib().oracle_fp32_Reduce_Backward(_ptr(dy), _ptr(dx), C.c_int(input_node_size), C.c_int(dy.shape[0]), C.c_int(frame_size), C.c_int(dy.shape[1]))
    return dx


def real_to_binary_forward(x, depth, points, frame_size, frame_mod=1, depth_mod=1, lo=0.0, hi=1.0, binarize=True, bit=False, y_stride=None):
    """x [depth * points, stride] -> y [depth * depth_mod * points, y_stride] (fp32, or words of packed bits): RealToBinary without a
    value generator (include/bb/RealToBinary.h:300-344)."""
    x = _c(x, np.float32)
    out_frames = frame_size * frame_mod
    if y_stride is None:
        y_stride = (out_frames + 31) // 32 if bit else out_frames
    y = np.zeros((depth * depth_mod * points, y_stride), np.int32 if bit else np.float32)
    f = lib().oracle_bit_RealToBinary_Forward if bit else lib().oracle_fp32_RealToBinary_Forward
    f(_ptr(x), _ptr(y), C.c_int(depth_mod), C.c_int(frame_mod), C.c_float(lo), C.c_float(hi), C.c_int(points), C.c_int(depth),
      C.c_int(frame_size), C.c_int(x.shape[1]), C.c_int(y_stride), C.c_int(int(binarize)))
    return y


def binary_to_real_forward(x, output_node_size, y_frame_size, frame_mux=1, bit=False, y_stride=None):
    """x [I, stride] (fp32 or packed bits; y_frame_size * frame_mux frames) -> y [O, y_stride]: the share of inputs > 0 among the
    I / O nodes and frame_mux frames that fold into an output element (include/bb/BinaryToReal.h:262-290)."""
    x = _c(x, np.int32 if bit else np.float32)
    y_stride = y_frame_size if y_stride is None else y_stride
    y = np.zeros((output_node_size, y_stride), np.float32)
    f = lib().oracle_bit_fp32_BinaryToReal_Forward if bit else lib().oracle_fp32_BinaryToReal_Forward
    f(_ptr(x), _ptr(y), C.c_int(x.shape[0] // output_node_size), C.c_int(frame_mux), C.c_int(output_node_size), C.c_int(x.shape[1]),
      C.c_int(y_frame_size), C.c_int(y_stride))
    return y


def binary_to_real_backward(dy, input_node_size, y_frame_size, frame_mux=1, x_stride=None):
    dy = _c(dy, np.float32)
    x_stride = y_frame_size * frame_mux if x_stride is None else x_stride
    dx = np.zeros((input_node_size, x_stride), np.float32)
    lib().oracle_fp32_BinaryToReal_Backward(_ptr(dy), _ptr(dx), C.c_int(input_node_size // dy.shape[0]), C.c_int(frame_mux), C.c_int(dy.shape[0]),
                                            C.c_int(x_stride), C.c_int(y_frame_size), C.c_int(dy.shape[1]))
    return dx


def binarize_forward(x, frame_size, th=0.0, low=-1.0, high=1.0, bit=False, y_stride=None):
    """y = x > th ? high : low (include/bb/Binarize.h:196-213), or the packed bits of x > th."""
    x = _c(x, np.float32)
    if bit:
        y_stride = (frame_size + 31) // 32 if y_stride is None else y_stride
        y = np.zeros((x.shape[0], y_stride), np.int32)
        lib().oracle_fp32_bit_Binarize_Forward(_ptr(x), _ptr(y), C.c_float(th), C.c_int(x.shape[0]), C.c_int(frame_size), C.c_int(x.shape[1]),
                                               C.c_int(y_stride))
        return y
    y = np.zeros_like(x)
    lib().oracle_fp32_Binarize_Forward(_ptr(x), _ptr(y), C.c_float(th), C.c_float(low), C.c_float(high), C.c_int(x.shape[0]), C.c_int(frame_size),
                                       C.c_int(x.shape[1]))
    return y


def hard_tanh_forward(x, frame_size, lo=-1.0, hi=1.0):
    x = _c(x, np.float32)
    y = np.zeros_like(x)
    lib().oracle_fp32_HardTanh_Forward(_ptr(x), _ptr(y), C.c_float(lo), C.c_float(hi), C.c_int(x.shape[0]), C.c_int(frame_size), C.c_int(x.shape[1]))
    return y


def hard_tanh_backward(x, dy, frame_size, lo=-1.0, hi=1.0):
    """dx = dy inside the open window (lo, hi), 0 elsewhere (include/bb/HardTanh.h:253-271); also the backward of Binarize."""
    x = _c(x, np.float32); dy = _c(dy, np.float32)
    dx = np.zeros_like(x)
    lib().oracle_fp32_HardTanh_Backward(_ptr(x), _ptr(dy), _ptr(dx), C.c_float(lo), C.c_float(hi), C.c_int(x.shape[0]), C.c_int(frame_size),
                                        C.c_int(x.shape[1]))
    return dx


def _pool_geometry(h, w, fh, fw):
    return (h + fh - 1) // fh, (w + fw - 1) // fw


def max_pooling_forward(x, c, h, w, fh, fw, frame_size):
    """fp32 x [c * h * w, stride] -> (y, argmax) [c * oh * ow, stride] (include/bb/MaxPooling.h:251-284)"""
    x = _c(x, np.float32)
    oh, ow = _pool_geometry(h, w, fh, fw)
    y = np.zeros((c * oh * ow, x.shape[1]), np.float32); arg = np.zeros((c * oh * ow, x.shape[1]), np.int32)
    lib().oracle_fp32_MaxPooling_Forward(_ptr(x), _ptr(y), _ptr(arg), C.c_int(fh), C.c_int(fw), C.c_int(w), C.c_int(h), C.c_int(ow), C.c_int(oh),
                                         C.c_int(c), C.c_int(frame_size), C.c_int(x.shape[1]))
    return y, arg


def max_pooling_backward(argmax, dy, c, h, w, fh, fw, frame_size):
    argmax = _c(argmax, np.int32); dy = _c(dy, np.float32)
    oh, ow = _pool_geometry(h, w, fh, fw)
    dx = np.zeros((c * h * w, dy.shape[1]), np.float32)
    lib().oracle_fp32_MaxPooling_Backward(_ptr(argmax), _ptr(dy), _ptr(dx), C.c_int(fh), C.c_int(fw), C.c_int(w), C.c_int(h), C.c_int(ow),
                                          C.c_int(oh), C.c_int(c), C.c_int(frame_size), C.c_int(dy.shape[1]))
    return dx


def bit_max_pooling_forward(xbits, c, h, w, fh, fw, frame_size):
    """packed x [c * h * w, words] -> packed y: the OR of each window (include/bb/MaxPooling.h:340-370)"""
    xbits = _c(xbits, np.int32)
    oh, ow = _pool_geometry(h, w, fh, fw)
    y = np.zeros((c * oh * ow, xbits.shape[1]), np.int32)
    lib().oracle_bit_MaxPooling_Forward(_ptr(xbits), _ptr(y), C.c_int(fh), C.c_int(fw), C.c_int(w), C.c_int(h), C.c_int(ow), C.c_int(oh),
                                        C.c_int(c), C.c_int(frame_size), C.c_int(xbits.shape[1]))
    return y


def bit_max_pooling_backward(xbits, dy, c, h, w, fh, fw, frame_size):
    """dy goes to the first set input of each window (include/bb/MaxPooling.h:551-579)"""
    xbits = _c(xbits, np.int32); dy = _c(dy, np.float32)
    oh, ow = _pool_geometry(h, w, fh, fw)
    dx = np.zeros((c * h * w, dy.shape[1]), np.float32)
    lib().oracle_bit_fp32_MaxPooling_Backward(_ptr(xbits), _ptr(dy), _ptr(dx), C.c_int(fh), C.c_int(fw), C.c_int(w), C.c_int(h), C.c_int(ow),
                                              C.c_int(oh), C.c_int(c), C.c_int(frame_size), C.c_int(xbits.shape[1]), C.c_int(dy.shape[1]))
    return dx


def up_sampling_forward(x, c, h, w, fh, fw, frame_size, fill=True, bit=False):
    """x [c * h * w, stride] (fp32 or packed words) -> y [c * h fh * w fw, stride] (include/bb/UpSampling.h:223-259)"""
    x = _c(x, np.int32 if bit else np.float32)
    y = np.zeros((c * h * fh * w * fw, x.shape[1]), x.dtype)
    f = lib().oracle_bit_UpSampling_Forward if bit else lib().oracle_fp32_UpSampling_Forward
    f(_ptr(x), _ptr(y), C.c_int(w), C.c_int(h), C.c_int(c), C.c_int(fw), C.c_int(fh), C.c_int(int(fill)), C.c_int(frame_size), C.c_int(x.shape[1]))
    return y


def up_sampling_backward(dy, c, h, w, fh, fw, frame_size, fill=True):
    dy = _c(dy, np.float32)
    dx = np.zeros((c * h * w, dy.shape[1]), np.float32)
    lib().oracle_fp32_UpSampling_Backward(_ptr(dy), _ptr(dx), C.c_int(w), C.c_int(h), C.c_int(c), C.c_int(fw), C.c_int(fh), C.c_int(int(fill)),
                                          C.c_int(frame_size), C.c_int(dy.shape[1]))
    return dx


def shuffle_forward(x, shuffle_unit):
    """Rows of 32-bit words (fp32 or packed bits alike), x [nodes, stride] -> y (include/bb/Shuffle.h:166-185)"""
    x = np.ascontiguousarray(x); assert x.dtype.itemsize == 4 and x.shape[0] % shuffle_unit == 0
    y = np.zeros_like(x)
    lib().oracle_Shuffle_Forward(_ptr(x), _ptr(y), C.c_int(shuffle_unit), C.c_int(x.shape[0]), C.c_int(x.shape[1]))
    return y


def shuffle_backward(dy, shuffle_unit):
    """include/bb/Shuffle.h:225-243"""
    dy = np.ascontiguousarray(dy); assert dy.dtype.itemsize == 4 and dy.shape[0] % shuffle_unit == 0
    dx = np.zeros_like(dy)
    lib().oracle_Shuffle_Backward(_ptr(dy), _ptr(dx), C.c_int(shuffle_unit), C.c_int(dy.shape[0]), C.c_int(dy.shape[1]))
    return dx


def loss_mean_squared_error(y, t, frame_size, batch_size=None, reduction_sum=False, loss=0.0):
    """-> (dy, loss accumulator): the reference's host loop (include/bb/LossMeanSquaredError.h:121-169) for one batch; `loss` is the
    accumulator before the batch.  The layer's loss is accumulator / frames seen (the accumulator itself with reduction "sum")."""
    y = _c(y, np.float32); t = _c(t, np.float32)
    nodes = y.shape[0]
    batch_size = frame_size if batch_size is None else batch_size
    grad_reduction = np.float32(1.0) if reduction_sum else np.float32(1.0) / np.float32(nodes * batch_size)
    loss_reduction = 1.0 if reduction_sum else 1.0 / nodes
    dy = np.zeros_like(y)
    acc = C.c_double(loss)
    lib().oracle_fp32_LossMeanSquaredError(_ptr(y), _ptr(t), _ptr(dy), C.byref(acc), C.c_int(nodes), C.c_int(frame_size), C.c_int(y.shape[1]),
                                           C.c_float(grad_reduction), C.c_double(loss_reduction))
    return dy, acc.value


def metrics_mean_squared_error(y, t, frame_size, accuracy=0.0):
    """-> the accumulator after the batch (include/bb/MetricsMeanSquaredError.h:66-85); the metric is accumulator / frames seen."""
    y = _c(y, np.float32); t = _c(t, np.float32)
    acc = C.c_double(accuracy)
    lib().oracle_fp32_MetricsMeanSquaredError(_ptr(y), _ptr(t), C.byref(acc), C.c_int(y.shape[0]), C.c_int(frame_size), C.c_int(y.shape[1]))
    return acc.value


def loss_t_sum(t, frame_size):
    t = _c(t, np.float32)
    f = lib().oracle_fp32_LossSoftmaxCrossEntropy_TSum
    f.restype = C.c_float
    return float(f(_ptr(t), C.c_int(t.shape[0]), C.c_int(frame_size), C.c_int(t.shape[1])))


def loss_softmax_cross_entropy(y, t, ch_size, pix_size, frame_size, t_sum=None):
    """y, t [ch*pix, stride] -> (dy [ch*pix, stride], loss_buf [frames] float64, t_sum).  The loss of the batch is
    -loss_buf.sum() / t_sum."""
    y = _c(y, np.float32); t = _c(t, np.float32)
    if t_sum is None:
        t_sum = loss_t_sum(t, frame_size)
    dy = np.zeros_like(y)
    loss_buf = np.zeros(frame_size, np.float64)
    lib().oracle_fp32_LossSoftmaxCrossEntropy(_ptr(y), _ptr(t), _ptr(dy), _ptr(loss_buf), C.c_float(t_sum), C.c_int(pix_size),
                                              C.c_int(ch_size), C.c_int(frame_size), C.c_int(y.shape[1]))
    return dy, loss_buf, t_sum


def metrics_categorical_accuracy(y, t, ch_size, pix_size, frame_size):
    """-> (accuracy_buf, category_buf) int32 [frames]; the metric of the batch is their sums' ratio."""
    y = _c(y, np.float32); t = _c(t, np.float32)
    acc = np.zeros(frame_size, np.int32); cat = np.zeros(frame_size, np.int32)
    lib().oracle_fp32_MetricsCategoricalAccuracy(_ptr(y), _ptr(t), _ptr(acc), _ptr(cat), C.c_int(pix_size), C.c_int(ch_size),
                                                 C.c_int(frame_size), C.c_int(y.shape[1]))
    return acc, cat


def stochastic_lut_forward(n, x, idx, W, frame_size, input_binary=False, lut_binarize=False, bias=0.25, simd=True):
    """fp32 x [I, stride] -> y [O, stride] (padding columns zero)."""
    x = _c(x, np.float32); idx = _c(idx, np.int32); W = _c(W, np.float32)
    O = idx.shape[0]; stride = x.shape[1]
    y = np.zeros((O, stride), np.float32)
    lib().oracle_fp32_StochasticLut_Forward(C.c_int(n), _ptr(x), _ptr(y), _ptr(idx), _ptr(W), C.c_int(O), C.c_int(frame_size),
                                            C.c_int(stride), C.c_int(int(input_binary)), C.c_int(int(lut_binarize)),
                                            C.c_float(bias), C.c_int(int(simd)))
    return y


def bit_stochastic_lut_forward(n, xbits, idx, W, frame_size, y_stride, lut_binarize=False, bias=0.25):
    xbits = _c(xbits, np.int32); idx = _c(idx, np.int32); W = _c(W, np.float32)
    O = idx.shape[0]
    y = np.zeros((O, y_stride), np.float32)
    lib().oracle_bit_fp32_StochasticLut_Forward(C.c_int(n), _ptr(xbits), _ptr(y), _ptr(idx), _ptr(W), C.c_int(O),
                                                C.c_int(frame_size), C.c_int(y_stride), C.c_int(xbits.shape[1]),
                                                C.c_int(int(lut_binarize)), C.c_float(bias))
    return y


def bit_bit_stochastic_lut_forward(n, xbits, idx, W, frame_size, lut_binarize=False, bias=0.25):
    xbits = _c(xbits, np.int32); idx = _c(idx, np.int32); W = _c(W, np.float32)
    O = idx.shape[0]
    y = np.zeros((O, xbits.shape[1]), np.int32)
    lib().oracle_bit_bit_fp32_StochasticLut_Forward(C.c_int(n), _ptr(xbits), _ptr(y), _ptr(idx), _ptr(W), C.c_int(O),
                                                    C.c_int(frame_size), C.c_int(xbits.shape[1]),
                                                    C.c_int(int(lut_binarize)), C.c_float(bias))
    return y


def stochastic_lut_backward(n, x, dy, idx, W, frame_size, dW_init=None, input_binary=False, lut_binarize=False,
                            bias=0.25, simd=True):
    """returns (dx [I, stride], dW [O, 2^n]); dW starts from dW_init (zeros when None)."""
    x = _c(x, np.float32); dy = _c(dy, np.float32); idx = _c(idx, np.int32); W = _c(W, np.float32)
    I, stride = x.shape; O = idx.shape[0]
    dx = np.zeros((I, stride), np.float32)
    dW = np.zeros((O, 1 << n), np.float32) if dW_init is None else _c(dW_init, np.float32).copy()
    lib().oracle_fp32_StochasticLut_Backward(C.c_int(n), _ptr(x), _ptr(dy), _ptr(dx), _ptr(idx), _ptr(W), _ptr(dW),
                                             C.c_int(I), C.c_int(O), C.c_int(frame_size), C.c_int(stride),
                                             C.c_int(int(input_binary)), C.c_int(int(lut_binarize)), C.c_float(bias),
                                             C.c_int(int(simd)))
    return dx, dW


def bit_stochastic_lut_backward(n, xbits, dy, idx, W, frame_size, dW_init=None, lut_binarize=False, bias=0.25):
    xbits = _c(xbits, np.int32); dy = _c(dy, np.float32); idx = _c(idx, np.int32); W = _c(W, np.float32)
    I = xbits.shape[0]; O = idx.shape[0]; stride = dy.shape[1]
    dx = np.zeros((I, stride), np.float32)
    dW = np.zeros((O, 1 << n), np.float32) if dW_init is None else _c(dW_init, np.float32).copy()
    lib().oracle_bit_fp32_StochasticLut_Backward(C.c_int(n), _ptr(xbits), _ptr(dy), _ptr(dx), _ptr(idx), _ptr(W), _ptr(dW),
                                                 C.c_int(I), C.c_int(O), C.c_int(frame_size), C.c_int(stride),
                                                 C.c_int(xbits.shape[1]), C.c_int(int(lut_binarize)), C.c_float(bias))
    return dx, dW


def differentiable_lut_forward_training(n, x, idx, W, frame_size, running_mean, running_var, gamma=0.3, beta=0.5,
                                        momentum=0.9, bias=0.25, lut_binarize=False, binary_mode=True):
    """fp32 x. returns (y, mean, rstd, running_mean, running_var)."""
    x = _c(x, np.float32); idx = _c(idx, np.int32); W = _c(W, np.float32)
    O = idx.shape[0]; stride = x.shape[1]
    y = np.zeros((O, stride), np.float32)
    mean = np.zeros(O, np.float32); rstd = np.zeros(O, np.float32)
    rm = _c(running_mean, np.float32).copy(); rv = _c(running_var, np.float32).copy()
    lib().oracle_fp32_DifferentiableLutN_ForwardTraining(
        C.c_int(n), _ptr(x), _ptr(y), _ptr(idx), _ptr(W), _ptr(mean), _ptr(rstd), _ptr(rm), _ptr(rv),
        C.c_float(gamma), C.c_float(beta), C.c_float(momentum), C.c_float(bias),
        C.c_int(O), C.c_int(frame_size), C.c_int(stride), C.c_int(int(lut_binarize)), C.c_int(int(binary_mode)))
    return y, mean, rstd, rm, rv


def bit_differentiable_lut_forward_training(n, xbits, idx, W, frame_size, running_mean, running_var, gamma=0.3, beta=0.5,
                                            momentum=0.9, bias=0.25, lut_binarize=False):
    xbits = _c(xbits, np.int32); idx = _c(idx, np.int32); W = _c(W, np.float32)
    O = idx.shape[0]; stride = xbits.shape[1]
    y = np.zeros((O, stride), np.int32)
    mean = np.zeros(O, np.float32); rstd = np.zeros(O, np.float32)
    rm = _c(running_mean, np.float32).copy(); rv = _c(running_var, np.float32).copy()
    lib().oracle_bit_fp32_DifferentiableLutN_ForwardTraining(
        C.c_int(n), _ptr(xbits), _ptr(y), _ptr(idx), _ptr(W), _ptr(mean), _ptr(rstd), _ptr(rm), _ptr(rv),
        C.c_float(gamma), C.c_float(beta), C.c_float(momentum), C.c_float(bias),
        C.c_int(O), C.c_int(frame_size), C.c_int(stride), C.c_int(int(lut_binarize)))
    return y, mean, rstd, rm, rv


def differentiable_lut_forward_inference(n, x, idx, W, frame_size, running_mean, running_var, gamma=0.3, beta=0.5,
                                         bias=0.25, lut_binarize=False, binary_mode=True):
    x = _c(x, np.float32); idx = _c(idx, np.int32); W = _c(W, np.float32)
    O = idx.shape[0]; stride = x.shape[1]
    y = np.zeros((O, stride), np.float32)
    rm = _c(running_mean, np.float32); rv = _c(running_var, np.float32)
    lib().oracle_fp32_DifferentiableLutN_ForwardInference(
        C.c_int(n), _ptr(x), _ptr(y), _ptr(idx), _ptr(W), _ptr(rm), _ptr(rv),
        C.c_float(gamma), C.c_float(beta), C.c_float(bias),
        C.c_int(O), C.c_int(frame_size), C.c_int(stride), C.c_int(int(lut_binarize)), C.c_int(int(binary_mode)))
    return y


def bit_differentiable_lut_forward_inference(n, xbits, idx, W, frame_size, running_mean, running_var, gamma=0.3,
                                             beta=0.5, bias=0.25, lut_binarize=False):
    xbits = _c(xbits, np.int32); idx = _c(idx, np.int32); W = _c(W, np.float32)
    O = idx.shape[0]; stride = xbits.shape[1]
    y = np.zeros((O, stride), np.int32)
    rm = _c(running_mean, np.float32); rv = _c(running_var, np.float32)
    lib().oracle_bit_fp32_DifferentiableLutN_ForwardInference(
        C.c_int(n), _ptr(xbits), _ptr(y), _ptr(idx), _ptr(W), _ptr(rm), _ptr(rv),
        C.c_float(gamma), C.c_float(beta), C.c_float(bias),
        C.c_int(O), C.c_int(frame_size), C.c_int(stride), C.c_int(int(lut_binarize)))
    return y


def differentiable_lut_forward_nobn(n, x, idx, W, frame_size, bias=0.25, lut_binarize=False, binary_mode=True):
    x = _c(x, np.float32); idx = _c(idx, np.int32); W = _c(W, np.float32)
    O = idx.shape[0]; stride = x.shape[1]
    y = np.zeros((O, stride), np.float32)
    lib().oracle_fp32_DifferentiableLutN_ForwardNoBn(
        C.c_int(n), _ptr(x), _ptr(y), _ptr(idx), _ptr(W), C.c_float(bias),
        C.c_int(O), C.c_int(frame_size), C.c_int(stride), C.c_int(int(lut_binarize)), C.c_int(int(binary_mode)))
    return y


def differentiable_lut_backward(n, x, dy, idx, W, frame_size, mean, rstd, dW_init=None, gamma=0.3, beta=0.5, bias=0.25,
                                lut_binarize=False, binary_mode=True):
    x = _c(x, np.float32); dy = _c(dy, np.float32); idx = _c(idx, np.int32); W = _c(W, np.float32)
    I, stride = x.shape; O = idx.shape[0]
    dx = np.zeros((I, stride), np.float32)
    dW = np.zeros((O, 1 << n), np.float32) if dW_init is None else _c(dW_init, np.float32).copy()
    lib().oracle_fp32_DifferentiableLutN_Backward(
        C.c_int(n), _ptr(x), _ptr(dy), _ptr(dx), _ptr(idx), _ptr(W), _ptr(dW), _ptr(_c(mean, np.float32)),
        _ptr(_c(rstd, np.float32)), C.c_float(gamma), C.c_float(beta), C.c_float(bias),
        C.c_int(I), C.c_int(O), C.c_int(frame_size), C.c_int(stride), C.c_int(int(lut_binarize)), C.c_int(int(binary_mode)))
    return dx, dW


def bit_differentiable_lut_backward(n, xbits, dy, idx, W, frame_size, mean, rstd, dW_init=None, gamma=0.3, beta=0.5,
                                    bias=0.25, lut_binarize=False):
    xbits = _c(xbits, np.int32); dy = _c(dy, np.float32); idx = _c(idx, np.int32); W = _c(W, np.float32)
    I = xbits.shape[0]; O = idx.shape[0]; stride = dy.shape[1]
    dx = np.zeros((I, stride), np.float32)
    dW = np.zeros((O, 1 << n), np.float32) if dW_init is None else _c(dW_init, np.float32).copy()
    lib().oracle_bit_fp32_DifferentiableLutN_Backward(
        C.c_int(n), _ptr(xbits), _ptr(dy), _ptr(dx), _ptr(idx), _ptr(W), _ptr(dW), _ptr(_c(mean, np.float32)),
        _ptr(_c(rstd, np.float32)), C.c_float(gamma), C.c_float(beta), C.c_float(bias),
        C.c_int(I), C.c_int(O), C.c_int(frame_size), C.c_int(stride), C.c_int(xbits.shape[1]), C.c_int(int(lut_binarize)))
    return dx, dW


def binary_lut6_forward(xbits, idx, table, frame_size, words=False):
    """packed x [I, stride_words] int32 -> packed y [O, stride_words]; bits of frames >= frame_size stay zero
    (generic loop) or are computed from the padding (words=True, the AVX2-shaped loop)."""
    xbits = _c(xbits, np.int32); idx = _c(idx, np.int32); table = _c(table, np.int32)
    O = idx.shape[0]; stride = xbits.shape[1]
    y = np.zeros((O, stride), np.int32)
    if words:
        lib().oracle_bit_BinaryLut6_Forward_words(_ptr(xbits), _ptr(y), _ptr(idx), _ptr(table), C.c_int(O),
                                                  C.c_int((frame_size + 31) // 32), C.c_int(stride))
    else:
        lib().oracle_bit_BinaryLut6_Forward(_ptr(xbits), _ptr(y), _ptr(idx), _ptr(table), C.c_int(O),
                                            C.c_int(frame_size), C.c_int(stride))
    return y


def reverse_table(n, idx, input_node_size):
    idx = _c(idx, np.int32)
    O = idx.shape[0]
    f = lib().oracle_ReverseTable
    f.restype = C.c_int
    stride = f(C.c_int(n), _ptr(idx), C.c_int(input_node_size), C.c_int(O), None, C.c_int(0))
    rev = np.zeros((input_node_size, stride), np.int32)
    f(C.c_int(n), _ptr(idx), C.c_int(input_node_size), C.c_int(O), _ptr(rev), C.c_int(rev.size))
    return rev


# ----------------------------------------------------------------------------------------------
#  the real reference headers (oracle/_ref/libbbref.so) — dense [nodes, frames] arrays, no stride
# ----------------------------------------------------------------------------------------------

def binary_lutn_forward(n, xbits, idx, table, frame_size):
    """BinaryLutN<n>, n = 2 .. 6: packed x [I, stride_words] -> packed y [O, stride_words]; table [O, (2^n + 31) // 32] words, entry i = bit
    i & 31 of word i >> 5; bits of frames >= frame_size stay zero (the reference's generic loop, include/bb/BinaryLutN.h:436-463)."""
    xbits = _c(xbits, np.int32); idx = _c(idx, np.int32); table = _c(table, np.int32)
    O = idx.shape[0]; stride = xbits.shape[1]
    assert idx.shape[1] == n and table.shape == (O, ((1 << n) + 31) // 32)
    y = np.zeros((O, stride), np.int32)
    lib().oracle_bit_BinaryLutN_Forward(C.c_int(n), _ptr(xbits), _ptr(y), _ptr(idx), _ptr(table), C.c_int(O), C.c_int(frame_size), C.c_int(stride))
    return y


def ref_stochastic_lut(n, x, idx, W, dy=None, dW_init=None, bit_input=False, binary_mode=False, lut_binarize=False,
                       host_simd=True, frame_size=None):
    """Runs bb::StochasticLutN<n,...>::Forward (+Backward). Returns dict(y, W, dx, dW)."""
    idx = _c(idx, np.int32); W = _c(W, np.float32).copy()
    O = idx.shape[0]
    if bit_input:
        x = _c(x, np.int32); I = x.shape[0]; F = frame_size
        assert x.shape[1] == (F + 31) // 32
    else:
        x = _c(x, np.float32); I, F = x.shape
    y = np.zeros((O, F), np.float32)
    dx = np.zeros((I, F), np.float32) if dy is not None else None
    dW = None
    if dy is not None:
        dy = _c(dy, np.float32)
        dW = np.zeros((O, 1 << n), np.float32) if dW_init is None else _c(dW_init, np.float32).copy()
    rc = ref().bbref_StochasticLut(C.c_int(n), C.c_int(int(bit_input)), C.c_int(I), C.c_int(O), C.c_int(F),
                                   _ptr(x), _ptr(idx), _ptr(W), _ptr(dy), _ptr(y), _ptr(dx), _ptr(dW),
                                   C.c_int(int(binary_mode)), C.c_int(int(lut_binarize)), C.c_int(int(host_simd)))
    assert rc == 0
    return dict(y=y, W=W, dx=dx, dW=dW)


def ref_differentiable_lut(n, x, idx, W, running_mean, running_var, dy=None, dW_init=None, bit_input=False,
                           gamma=0.3, beta=0.5, momentum=0.9, batch_norm=True, binary_mode=True, lut_binarize=False,
                           train=True, frame_size=None):
    idx = _c(idx, np.int32); W = _c(W, np.float32).copy()
    O = idx.shape[0]
    if bit_input:
        x = _c(x, np.int32); I = x.shape[0]; F = frame_size
        y = np.zeros((O, (F + 31) // 32), np.int32)
    else:
        x = _c(x, np.float32); I, F = x.shape
        y = np.zeros((O, F), np.float32)
    dx = np.zeros((I, F), np.float32) if dy is not None else None
    dW = None
    if dy is not None:
        dy = _c(dy, np.float32)
        dW = np.zeros((O, 1 << n), np.float32) if dW_init is None else _c(dW_init, np.float32).copy()
    mean = np.zeros(O, np.float32); rstd = np.zeros(O, np.float32)
    rm = _c(running_mean, np.float32).copy(); rv = _c(running_var, np.float32).copy()
    rc = ref().bbref_DifferentiableLut(C.c_int(n), C.c_int(int(bit_input)), C.c_int(I), C.c_int(O), C.c_int(F),
                                       _ptr(x), _ptr(idx), _ptr(W), _ptr(dy), _ptr(y), _ptr(dx), _ptr(dW),
                                       _ptr(mean), _ptr(rstd), _ptr(rm), _ptr(rv),
                                       C.c_float(gamma), C.c_float(beta), C.c_float(momentum),
                                       C.c_int(int(batch_norm)), C.c_int(int(binary_mode)), C.c_int(int(lut_binarize)),
                                       C.c_int(int(train)))
    assert rc == 0
    return dict(y=y, W=W, dx=dx, dW=dW, mean=mean, rstd=rstd, running_mean=rm, running_var=rv)


def ref_binary_lut6(xbits, idx, table, frame_size, host_simd=True):
    xbits = _c(xbits, np.int32); idx = _c(idx, np.int32); table = _c(table, np.int32)
    I = xbits.shape[0]; O = idx.shape[0]
    assert xbits.shape[1] == (frame_size + 31) // 32
    y = np.zeros((O, xbits.shape[1]), np.int32)
    rc = ref().bbref_BinaryLut6(C.c_int(I), C.c_int(O), C.c_int(frame_size), _ptr(xbits), _ptr(idx), _ptr(table), _ptr(y),
                                C.c_int(int(host_simd)))
    assert rc == 0
    return y


def ref_binary_lutn(n, xbits, idx, table, frame_size):
    """bb::BinaryLutN<n, Bit>::Forward of the reference (host path), n = 2 .. 6; dense packed arrays [rows, ceil(frames / 32)]"""
    xbits = _c(xbits, np.int32); idx = _c(idx, np.int32); table = _c(table, np.int32)
    I = xbits.shape[0]; O = idx.shape[0]
    assert xbits.shape[1] == (frame_size + 31) // 32 and idx.shape[1] == n
    y = np.zeros((O, xbits.shape[1]), np.int32)
    rc = ref().bbref_BinaryLutN(C.c_int(n), C.c_int(I), C.c_int(O), C.c_int(frame_size), _ptr(xbits), _ptr(idx), _ptr(table), _ptr(y))
    assert rc == 0
    return y


def ref_wiring6(kind, input_shape, output_shape, seed, policy):
    """Wiring that the reference gives a 6-input layer from a seed and a policy string.  kind 0: the connection table of
    StochasticLutN / DifferentiableLutN; kind 1: BinaryLutN (also returns its random truth tables [O][2])."""
    ins = np.asarray(input_shape, np.int64); outs = np.asarray(output_shape, np.int64)
    O = int(np.prod(outs))
    idx = np.zeros((O, 6), np.int32); table = np.zeros((O, 2), np.int32)
    f = ref().bbref_Wiring6
    f.restype = C.c_int
    rc = f(C.c_int(kind), C.c_int(len(ins)), _ptr(ins), _ptr(outs), C.c_uint64(seed), C.c_char_p(policy.encode()), _ptr(idx), _ptr(table))
    assert rc == 0
    return (idx, table) if kind == 1 else idx


def ref_dump_container_object(kind, c, h, w, fh, fw, ys=1, xs=1, same=False, border_mode="reflect_101", o1=16, o2=8, seed=1, name=""):
    """Bytes of a container object as the reference writes it.  kind 0: Convolution2d over one DifferentiableLut6 (o2 nodes);
    1: Convolution2d over a Sequential of two (o1, o2); 2: that Sequential alone; 3: ConvolutionIm2Col; 4: ConvolutionCol2Im
    (image h x w, o2 channels)."""
    f = ref().bbref_DumpContainerObject
    f.restype = C.c_long
    out = np.zeros(1 << 22, np.uint8)
    n = f(C.c_int(kind), C.c_int(c), C.c_int(h), C.c_int(w), C.c_int(fh), C.c_int(fw), C.c_int(ys), C.c_int(xs), C.c_int(int(same)),
          C.c_char_p(border_mode.encode()), C.c_int(o1), C.c_int(o2), C.c_int(seed), C.c_char_p(name.encode()), _ptr(out), C.c_long(out.size))
    assert n > 0, n
    return out[:n].copy()


def ref_reload_container_object(data):
    """The reference loads the object (rebuilding it from the type names in the stream) and dumps it again; None if it cannot."""
    data = _c(data, np.uint8)
    f = ref().bbref_ReloadContainerObject
    f.restype = C.c_long
    out = np.zeros(max(1 << 22, 2 * data.size), np.uint8)
    n = f(_ptr(data), C.c_long(data.size), _ptr(out), C.c_long(out.size))
    return out[:n].copy() if n > 0 else None


def ref_stochastic_bn(x, running_mean, running_var, gamma, beta, momentum, train=True, dy=None, name="", want_object=False):
    """The reference's StochasticBatchNormalization<float> (generic host path) on dense [nodes, frames] arrays ->
    dict(y, mean, rstd, running_mean, running_var, dx, object)."""
    x = _c(x, np.float32)
    nodes, frames = x.shape
    y = np.zeros_like(x)
    rm = _c(running_mean, np.float32).copy(); rv = _c(running_var, np.float32).copy()
    mean = np.zeros(nodes, np.float32); rstd = np.zeros(nodes, np.float32)
    dx = None
    if dy is not None:
        dy = _c(dy, np.float32); dx = np.zeros_like(x)
    out = np.zeros((1 << 16) + 16 * nodes, np.uint8) if want_object else None
    f = ref().bbref_StochasticBatchNormalization
    f.restype = C.c_long
    n = f(C.c_int(nodes), C.c_int(frames), C.c_float(momentum), C.c_float(gamma), C.c_float(beta), C.c_int(int(train)), _ptr(x), _ptr(rm),
          _ptr(rv), _ptr(y), _ptr(mean), _ptr(rstd), _ptr(dy), _ptr(dx), C.c_char_p(name.encode()), _ptr(out),
          C.c_long(out.size if want_object else 0))
    assert n >= 0, n
    return dict(y=y, mean=mean, rstd=rstd, running_mean=rm, running_var=rv, dx=dx, object=out[:n].copy() if want_object else None)


def ref_reverse_table6(idx, input_node_size):
    idx = _c(idx, np.int32)
    O = idx.shape[0]
    f = ref().bbref_ReverseTable6
    f.restype = C.c_int
    stride = f(C.c_int(input_node_size), C.c_int(O), _ptr(idx), None, C.c_int(0))
    rev = np.zeros((input_node_size, stride), np.int32)
    f(C.c_int(input_node_size), C.c_int(O), _ptr(idx), _ptr(rev), C.c_int(rev.size))
    return rev


# ----------------------------------------------------------------------------------------------
#  timed CPU baselines (used by bench.py only)
# ----------------------------------------------------------------------------------------------

def ref_adam_steps(param, grads, learning_rate=0.001, beta1=0.9, beta2=0.999):
    """bb::OptimizerAdam<float> of the reference (host path): param after len(grads) updates."""
    p = _c(param, np.float32).copy()
    g = _c(np.stack([np.asarray(x, np.float32).ravel() for x in grads]), np.float32)
    rc = ref().bbref_OptimizerAdam(C.c_int(p.size), C.c_int(g.shape[0]), _ptr(p), _ptr(g), C.c_float(learning_rate),
                                   C.c_float(beta1), C.c_float(beta2))
    assert rc == 0
    return p


def ref_vector_op(name, src0, src1=None, a=0.0, b=0.0, c=0.0, d=0.0):
    src0 = _c(src0, np.float32)
    src1 = None if src1 is None else _c(src1, np.float32)
    dst = np.empty_like(src0)
    rc = ref().bbref_Vector_op(C.c_int(_VEC_OPS[name]), _ptr(dst), _ptr(src0), _ptr(src1), C.c_float(a), C.c_float(b),
                               C.c_float(c), C.c_float(d), C.c_int(src0.size))
    assert rc == 0
    return dst


def ref_im2col(x, c, h, w, frames, fh, fw, ys=1, xs=1, padding="valid", border="reflect_101", dy=None, bit=False):
    """The reference's ConvolutionIm2Col (host path): returns (y, dx or None).  Dense arrays: fp32 [nodes, frames] or
    packed [nodes, ceil(frames/32)]."""
    oh, ow, _, _ = im2col_geometry(h, w, fh, fw, ys, xs, padding)
    of = frames * oh * ow
    if bit:
        x = _c(x, np.int32); y = np.zeros((c * fh * fw, (of + 31) // 32), np.int32)
    else:
        x = _c(x, np.float32); y = np.zeros((c * fh * fw, of), np.float32)
    dx = None
    if dy is not None:
        dy = _c(dy, np.float32); dx = np.zeros((c * h * w, frames), np.float32)
    hw = (C.c_int * 2)()
    got = ref().bbref_Im2Col(C.c_int(int(bit)), C.c_int(c), C.c_int(h), C.c_int(w), C.c_int(frames), C.c_int(fh), C.c_int(fw),
                             C.c_int(ys), C.c_int(xs), padding.encode(), border.encode(), _ptr(x), _ptr(y), _ptr(dy), _ptr(dx), hw)
    assert got == of and (hw[0], hw[1]) == (oh, ow)
    return y, dx


def ref_col2im(x, c, h, w, frames, dy=None, bit=False):
    if bit:
        x = _c(x, np.int32); y = np.zeros((c * h * w, (frames + 31) // 32), np.int32)
    else:
        x = _c(x, np.float32); y = np.zeros((c * h * w, frames), np.float32)
    dx = None
    if dy is not None:
        dy = _c(dy, np.float32); dx = np.zeros((c, frames * h * w), np.float32)
    assert ref().bbref_Col2Im(C.c_int(int(bit)), C.c_int(c), C.c_int(h), C.c_int(w), C.c_int(frames), _ptr(x), _ptr(y), _ptr(dy), _ptr(dx)) == 0
    return y, dx


def ref_stochastic_maxpool2x2(x, c, h, w, frames, dy=None):
    x = _c(x, np.float32)
    oh, ow = (h + 1) // 2, (w + 1) // 2
    y = np.zeros((c * oh * ow, frames), np.float32)
    dx = None
    if dy is not None:
        dy = _c(dy, np.float32); dx = np.zeros((c * h * w, frames), np.float32)
    assert ref().bbref_StochasticMaxPooling2x2(C.c_int(c), C.c_int(h), C.c_int(w), C.c_int(frames), _ptr(x), _ptr(y), _ptr(dy), _ptr(dx)) == 0
    return y, dx


def ref_average_lut(x, idx, input_node_size, frames, bit=False, binarize_input=False, binarize_output=True, dy=None):
    """The reference's AverageLut host path on dense [nodes, frames] (or [nodes, words]) arrays -> (y, dx)."""
    idx = _c(idx, np.int32)
    O, n = idx.shape
    if bit:
        x = _c(x, np.int32); y = np.zeros((O, (frames + 31) // 32), np.int32)
    else:
        x = _c(x, np.float32); y = np.zeros((O, frames), np.float32)
    dx = None
    if dy is not None:
        dy = _c(dy, np.float32); dx = np.zeros((input_node_size, frames), np.float32)
    assert ref().bbref_AverageLut(C.c_int(int(bit)), C.c_int(n), C.c_int(input_node_size), C.c_int(O), C.c_int(frames), _ptr(x), _ptr(idx),
                                  C.c_int(int(binarize_input)), C.c_int(int(binarize_output)), _ptr(y), _ptr(dy), _ptr(dx)) == 0
    return y, dx


def ref_max_lut(x, idx, input_node_size, frames, bit=False, binarize_input=False, binarize_output=True, dy=None, name="", want_object=False):
    """The reference's MaxLut host path on dense [nodes, frames] (or [nodes, words]) arrays -> (y, dx, object bytes)."""
    idx = _c(idx, np.int32)
    O, n = idx.shape
    if bit:
        x = _c(x, np.int32); y = np.zeros((O, (frames + 31) // 32), np.int32)
    else:
        x = _c(x, np.float32); y = np.zeros((O, frames), np.float32)
    dx = None
    if dy is not None:
        dy = _c(dy, np.float32); dx = np.zeros((input_node_size, frames), np.float32)
    out = np.zeros((1 << 16) + 8 * idx.size, np.uint8) if want_object else None
    f = ref().bbref_MaxLut
    f.restype = C.c_long
    r = f(C.c_int(int(bit)), C.c_int(n), C.c_int(input_node_size), C.c_int(O), C.c_int(frames), _ptr(x), _ptr(idx),
          C.c_int(int(binarize_input)), C.c_int(int(binarize_output)), _ptr(y), _ptr(dy), _ptr(dx), C.c_char_p(name.encode()), _ptr(out),
          C.c_long(out.size if want_object else 0))
    assert r >= 0, r
    return y, dx, (out[:r].copy() if want_object else None)


def ref_average_lut_object(idx, input_node_size, bit=False, binarize_input=False, binarize_output=True, name=""):
    """Bytes of an AverageLut layer with the given wiring as the reference's DumpObject writes it."""
    idx = _c(idx, np.int32)
    O, n = idx.shape
    out = np.zeros((1 << 16) + 8 * idx.size, np.uint8)
    f = ref().bbref_AverageLutObject
    f.restype = C.c_long
    r = f(C.c_int(int(bit)), C.c_int(n), C.c_int(input_node_size), C.c_int(O), _ptr(idx), C.c_int(int(binarize_input)),
          C.c_int(int(binarize_output)), C.c_char_p(name.encode()), _ptr(out), C.c_long(out.size))
    assert r > 0, r
    return out[:r].copy()


def ref_reduce(x, output_node_size, frames, bit=False, integration_size=0, dy=None, name="", want_object=False):
    """The reference's Reduce host path on dense [nodes, frames] (or [nodes, words]) arrays -> (y, dx, object bytes)."""
    x = _c(x, np.int32 if bit else np.float32)
    I = x.shape[0]
    y = np.zeros((output_node_size, frames), np.float32)
    dx = None
    if dy is not None:
        dy = _c(dy, np.float32); dx = np.zeros((I, frames), np.float32)
    out = np.zeros(1 << 16, np.uint8) if want_object else None
    f = ref().bbref_Reduce
    f.restype = C.c_long
    r = f(C.c_int(int(bit)), C.c_int(I), C.c_int(output_node_size), C.c_int(frames), C.c_int(integration_size), _ptr(x), _ptr(y), _ptr(dy),
          _ptr(dx), C.c_char_p(name.encode()), _ptr(out), C.c_long(out.size if want_object else 0))
    assert r >= 0, r
    return y, dx, (out[:r].copy() if want_object else None)


def ref_real_to_binary(x, depth, points, frames, frame_mod=1, depth_mod=1, lo=0.0, hi=1.0, binary_mode=True, bit=False, name="",
                       want_object=False):
    """The reference's RealToBinary host path (no value generator) on a dense [depth * points, frames] array -> (y, object bytes);
    y is [depth * depth_mod * points, frames * frame_mod] fp32, or rows of packed words."""
    x = _c(x, np.float32)
    out_nodes, out_frames = depth * depth_mod * points, frames * frame_mod
    y = np.zeros((out_nodes, (out_frames + 31) // 32), np.int32) if bit else np.zeros((out_nodes, out_frames), np.float32)
    out = np.zeros(1 << 16, np.uint8) if want_object else None
    f = ref().bbref_RealToBinary
    f.restype = C.c_long
    r = f(C.c_int(int(bit)), C.c_int(depth), C.c_int(points), C.c_int(frames), C.c_int(frame_mod), C.c_int(depth_mod), C.c_float(lo),
          C.c_float(hi), C.c_int(int(binary_mode)), _ptr(x), _ptr(y), C.c_char_p(name.encode()), _ptr(out),
          C.c_long(out.size if want_object else 0))
    assert r >= 0, r
    return y, (out[:r].copy() if want_object else None)


def ref_binary_to_real(x, output_node_size, frames, frame_mux=1, bit=False, dy=None, name="", want_object=False):
    """The reference's BinaryToReal host path; x [I, frames] fp32 or [I, words] bits -> (y [O, frames / frame_mux], dx, object bytes)."""
    x = _c(x, np.int32 if bit else np.float32)
    I = x.shape[0]
    y = np.zeros((output_node_size, frames // frame_mux), np.float32)
    dx = None
    if dy is not None:
        dy = _c(dy, np.float32); dx = np.zeros((I, frames), np.float32)
    out = np.zeros(1 << 16, np.uint8) if want_object else None
    f = ref().bbref_BinaryToReal
    f.restype = C.c_long
    r = f(C.c_int(int(bit)), C.c_int(I), C.c_int(output_node_size), C.c_int(frames), C.c_int(frame_mux), _ptr(x), _ptr(y), _ptr(dy), _ptr(dx),
          C.c_char_p(name.encode()), _ptr(out), C.c_long(out.size if want_object else 0))
    assert r >= 0, r
    return y, dx, (out[:r].copy() if want_object else None)


def ref_activation(kind, x, frames, bit=False, th=0.0, low=-1.0, high=1.0, lo=-1.0, hi=1.0, dy=None, name="", want_object=False):
    """The reference's Binarize (kind "binarize"), HardTanh ("hard_tanh") or HardTanh in binary mode ("hard_tanh_binary") host paths
    on a dense [nodes, frames] array -> (y, dx, object bytes); y is packed words where the layer's output type is Bit."""
    x = _c(x, np.float32)
    nodes = x.shape[0]
    y = np.zeros((nodes, (frames + 31) // 32), np.int32) if bit else np.zeros((nodes, frames), np.float32)
    dx = None
    if dy is not None:
        dy = _c(dy, np.float32); dx = np.zeros((nodes, frames), np.float32)
    out = np.zeros(1 << 16, np.uint8) if want_object else None
    f = ref().bbref_Activation
    f.restype = C.c_long
    r = f(C.c_int({"binarize": 0, "hard_tanh": 1, "hard_tanh_binary": 2}[kind]), C.c_int(int(bit)), C.c_int(nodes), C.c_int(frames),
          C.c_float(th), C.c_float(low), C.c_float(high), C.c_float(lo), C.c_float(hi), _ptr(x), _ptr(y), _ptr(dy), _ptr(dx),
          C.c_char_p(name.encode()), _ptr(out), C.c_long(out.size if want_object else 0))
    assert r >= 0, r
    return y, dx, (out[:r].copy() if want_object else None)


def ref_dump_binary_modulation_object(input_nodes, o1, o2, train_mod, infer_mod=0, depth_mod=1, bit=False, seed=1, run_inference=False, name=""):
    """The bytes of a BinaryModulation around a list of two DifferentiableLut6 layers as the reference's DumpObject writes them."""
    out = np.zeros(1 << 22, np.uint8)
    f = ref().bbref_DumpBinaryModulationObject
    f.restype = C.c_long
    r = f(C.c_int(int(bit)), C.c_int(input_nodes), C.c_int(o1), C.c_int(o2), C.c_int(train_mod), C.c_int(infer_mod), C.c_int(depth_mod),
          C.c_int(seed), C.c_int(int(run_inference)), C.c_char_p(name.encode()), _ptr(out), C.c_long(out.size))
    assert r > 0, r
    return out[:r].copy()


def ref_dump_discrete_lut_object(input_nodes, output_nodes, bit=False, seed=1, batch_norm=True, memory_saving=False, name=""):
    """The bytes of a DifferentiableLutDiscrete6 (StochasticLut6 -> StochasticBatchNormalization -> HardTanh) as the reference writes them."""
    out = np.zeros(1 << 22, np.uint8)
    f = ref().bbref_DumpDiscreteLutObject
    f.restype = C.c_long
    r = f(C.c_int(int(bit)), C.c_int(input_nodes), C.c_int(output_nodes), C.c_int(seed), C.c_int(int(batch_norm)), C.c_int(int(memory_saving)),
          C.c_char_p(name.encode()), _ptr(out), C.c_long(out.size))
    assert r > 0, r
    return out[:r].copy()


def ref_max_pooling(x, c, h, w, fh, fw, frames, bit=False, dy=None, name="", want_object=False):
    """The reference's MaxPooling host path on dense arrays -> (y, dx, object bytes); x [c * h * w, frames] fp32 or [.., words] bits."""
    x = _c(x, np.int32 if bit else np.float32)
    oh, ow = _pool_geometry(h, w, fh, fw)
    O = c * oh * ow
    y = np.zeros((O, (frames + 31) // 32), np.int32) if bit else np.zeros((O, frames), np.float32)
    dx = None
    if dy is not None:
        dy = _c(dy, np.float32); dx = np.zeros((c * h * w, frames), np.float32)
    out = np.zeros(1 << 16, np.uint8) if want_object else None
    f = ref().bbref_MaxPooling
    f.restype = C.c_long
    r = f(C.c_int(int(bit)), C.c_int(c), C.c_int(h), C.c_int(w), C.c_int(fh), C.c_int(fw), C.c_int(frames), _ptr(x), _ptr(y), _ptr(dy), _ptr(dx),
          C.c_char_p(name.encode()), _ptr(out), C.c_long(out.size if want_object else 0))
    assert r >= 0, r
    return y, dx, (out[:r].copy() if want_object else None)


def ref_up_sampling(x, c, h, w, fh, fw, frames, fill=True, bit=False, dy=None, name="", want_object=False):
    """The reference's UpSampling host path on dense arrays -> (y, dx, object bytes)."""
    x = _c(x, np.int32 if bit else np.float32)
    O = c * h * fh * w * fw
    y = np.zeros((O, (frames + 31) // 32), np.int32) if bit else np.zeros((O, frames), np.float32)
    dx = None
    if dy is not None:
        dy = _c(dy, np.float32); dx = np.zeros((c * h * w, frames), np.float32)
    out = np.zeros(1 << 16, np.uint8) if want_object else None
    f = ref().bbref_UpSampling
    f.restype = C.c_long
    r = f(C.c_int(int(bit)), C.c_int(c), C.c_int(h), C.c_int(w), C.c_int(fh), C.c_int(fw), C.c_int(int(fill)), C.c_int(frames), _ptr(x), _ptr(y),
          _ptr(dy), _ptr(dx), C.c_char_p(name.encode()), _ptr(out), C.c_long(out.size if want_object else 0))
    assert r >= 0, r
    return y, dx, (out[:r].copy() if want_object else None)


def ref_shuffle(x, shuffle_unit, frames, bit=False, dy=None, name="", want_object=False):
    """The reference's Shuffle host path on dense arrays (fp32 [nodes, frames] or packed words) -> (y, dx, object bytes)."""
    dt = np.int32 if bit else np.float32
    x = _c(x, dt)
    y = np.zeros_like(x)
    dx = None
    if dy is not None:
        dy = _c(dy, dt); dx = np.zeros_like(x)
    out = np.zeros(1 << 16, np.uint8) if want_object else None
    f = ref().bbref_Shuffle
    f.restype = C.c_long
    r = f(C.c_int(int(bit)), C.c_int(shuffle_unit), C.c_int(x.shape[0]), C.c_int(frames), _ptr(x), _ptr(y), _ptr(dy), _ptr(dx),
          C.c_char_p(name.encode()), _ptr(out), C.c_long(out.size if want_object else 0))
    assert r >= 0, r
    return y, dx, (out[:r].copy() if want_object else None)


def ref_mean_squared_error(y, t, frames, batches=1, reduction_sum=False):
    """The reference's LossMeanSquaredError and MetricsMeanSquaredError host paths over `batches` batches of `frames` frames held side
    by side in y and t -> (dy, loss, metric)."""
    y = _c(y, np.float32); t = _c(t, np.float32)
    assert y.shape[1] == frames * batches
    dy = np.zeros_like(y)
    loss = C.c_double(0); metric = C.c_double(0)
    assert ref().bbref_MeanSquaredError(C.c_int(y.shape[0]), C.c_int(frames), C.c_int(batches), C.c_int(int(reduction_sum)), _ptr(y), _ptr(t),
                                        _ptr(dy), C.byref(loss), C.byref(metric)) == 0
    return dy, loss.value, metric.value


def ref_loss_and_accuracy(y, t, ch_size, pix_size, frames):
    """The reference's LossSoftmaxCrossEntropy and MetricsCategoricalAccuracy host paths -> (dy, loss, metric)."""
    y = _c(y, np.float32); t = _c(t, np.float32)
    dy = np.zeros((ch_size * pix_size, frames), np.float32)
    loss = C.c_double(0); metric = C.c_double(0)
    assert ref().bbref_LossAndAccuracy(C.c_int(ch_size), C.c_int(pix_size), C.c_int(frames), _ptr(y), _ptr(t), _ptr(dy),
                                       C.byref(loss), C.byref(metric)) == 0
    return dy, loss.value, metric.value


LUT_OBJECT_KINDS = {"stochastic": 0, "differentiable": 1, "binary": 2}


def ref_dump_lut_object(kind, bit, input_nodes, idx, params, mean=None, var=None, flags=0, scalars=(0.9, 0.3, 0.5), name=""):
    """Bytes of a 6-input LUT layer serialized by the reference's own DumpObject.  params: W [O, 64] float32, or the truth
    table [O, 2] int32 for kind "binary".  flags: 1 = binary, 2 = lut_binarize, 4 = batch_norm."""
    idx = _c(idx, np.int32)
    params = _c(params, np.int32 if kind == "binary" else np.float32)
    O = idx.shape[0]
    mean = _c(mean if mean is not None else np.zeros(O), np.float32)
    var = _c(var if var is not None else np.ones(O), np.float32)
    sc = _c(scalars, np.float32)
    cap = 4096 + 64 * idx.nbytes + 2 * params.nbytes
    out = np.zeros(cap, np.uint8)
    f = ref().bbref_DumpLutObject
    f.restype = C.c_long
    n = f(C.c_int(LUT_OBJECT_KINDS[kind]), C.c_int(int(bit)), C.c_int(input_nodes), C.c_int(O), _ptr(idx), _ptr(params), _ptr(mean), _ptr(var),
          C.c_int(flags), _ptr(sc), C.c_char_p(name.encode()), _ptr(out), C.c_long(cap))
    assert n > 0, n
    return out[:n].tobytes()


def ref_load_lut_object(kind, bit, data, output_nodes):
    """A serialized layer read by the reference's own LoadObject -> dict(input_nodes, idx, params, mean, var, name)."""
    buf = np.frombuffer(data, np.uint8).copy()
    idx = np.zeros((output_nodes, 6), np.int32)
    params = np.zeros((output_nodes, 2), np.int32) if kind == "binary" else np.zeros((output_nodes, 64), np.float32)
    mean = np.zeros(output_nodes, np.float32); var = np.zeros(output_nodes, np.float32)
    name = C.create_string_buffer(256)
    I = ref().bbref_LoadLutObject(C.c_int(LUT_OBJECT_KINDS[kind]), C.c_int(int(bit)), _ptr(buf), C.c_long(buf.size), C.c_int(output_nodes),
                                  _ptr(idx), _ptr(params), _ptr(mean), _ptr(var), name, C.c_int(256))
    assert I >= 0, I
    return dict(input_nodes=I, idx=idx, params=params, mean=mean, var=var, name=name.value.decode())


def time_stochastic_lut6(x, dy, idx, W, reps=3, use_ref=None):
    """Seconds per StochasticLut6 forward+backward on the host, one value per repetition (after one warm-up).
    use_ref=True times the reference's own AVX2/OpenMP path, False the C restatement; None picks the reference when built."""
    x = _c(x, np.float32); dy = _c(dy, np.float32); idx = _c(idx, np.int32); W = _c(W, np.float32)
    I, F = x.shape; O = idx.shape[0]
    secs = np.zeros(reps, np.float64)
    if use_ref is None:
        use_ref = have_ref()
    if use_ref:
        rc = ref().bbref_StochasticLut6_Time(C.c_int(I), C.c_int(O), C.c_int(F), _ptr(x), _ptr(idx), _ptr(W), _ptr(dy),
                                             C.c_int(0), C.c_int(reps), _ptr(secs))
        assert rc == 0
    else:
        lib().oracle_fp32_StochasticLut6_Time(_ptr(x), _ptr(dy), _ptr(idx), _ptr(W), C.c_int(I), C.c_int(O), C.c_int(F),
                                              C.c_int(reps), _ptr(secs))
    return secs, ("reference" if use_ref else "port")
