"""Functional layer over the C ABI: torch device tensors in, torch device tensors out.

Every function is a direct call of one entry point of include/bbhip.h on the current torch stream.  Buffers follow
the FrameBuffer layout: ``[nodes, stride]`` float32 rows (stride >= frames) or ``[nodes, stride_words]`` int32 rows of
packed bits.  Nothing here has a CPU fallback: without the built library, or off a GPU, calls raise.
"""
import torch

from . import capi
from .capi import check, lib, ptr, stream_ptr


def _dev(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise capi.BbhipError("bbhip ops need device tensors")
        if t is not None and not t.is_contiguous():
            raise capi.BbhipError("bbhip ops need contiguous tensors")


def set_dx_mode(mode):
    """0: deterministic dx, input-centric re-evaluation through the reverse table (default); 1: fp32 atomics;
    2: the reference's scheme (per-connection gradients in dx_tmp, summed through the reverse table)."""
    lib().bbhip_SetDxMode(int(mode))


def vector_clamp_(t, lo=0.0, hi=1.0):
    _dev(t)
    check(lib().bbhip_fp32_Vector_clamp(ptr(t), ptr(t), lo, hi, t.numel(), stream_ptr()))
    return t


def vector_set_(t, value):
    _dev(t)
    check(lib().bbhip_fp32_Vector_set(ptr(t), value, t.numel(), stream_ptr()))
    return t


def _out(dst, like):
    return torch.empty_like(like) if dst is None else dst


def vector_add_ex(src0, src1, a=1.0, b=1.0, c=0.0, out=None):
    """a * src0 + b * src1 + c"""
    dst = _out(out, src0); _dev(src0, src1, dst)
    check(lib().bbhip_fp32_Vector_add_ex(ptr(dst), ptr(src0), ptr(src1), a, b, c, src0.numel(), stream_ptr()))
    return dst


def vector_mul_ex(src0, src1, a=1.0, b=0.0, out=None):
    """a * src0 * src1 + b"""
    dst = _out(out, src0); _dev(src0, src1, dst)
    check(lib().bbhip_fp32_Vector_mul_ex(ptr(dst), ptr(src0), ptr(src1), a, b, src0.numel(), stream_ptr()))
    return dst


def vector_div_ex(src0, src1, a=1.0, b=0.0, c=1.0, d=0.0, out=None):
    """(a * src0 + b) / (c * src1 + d)"""
    dst = _out(out, src0); _dev(src0, src1, dst)
    check(lib().bbhip_fp32_Vector_div_ex(ptr(dst), ptr(src0), ptr(src1), a, b, c, d, src0.numel(), stream_ptr()))
    return dst


def vector_unary(name, src, out=None):
    """name in {"sqrt", "exp"}"""
    dst = _out(out, src); _dev(src, dst)
    check(getattr(lib(), "bbhip_fp32_Vector_" + name)(ptr(dst), ptr(src), src.numel(), stream_ptr()))
    return dst


def vector_minmax(name, src0, src1, out=None):
    """name in {"min", "max"}; src1 is a tensor or a Python float (the *_v entry points)"""
    dst = _out(out, src0)
    if isinstance(src1, torch.Tensor):
        _dev(src0, src1, dst)
        check(getattr(lib(), "bbhip_fp32_Vector_" + name)(ptr(dst), ptr(src0), ptr(src1), src0.numel(), stream_ptr()))
    else:
        _dev(src0, dst)
        check(getattr(lib(), "bbhip_fp32_Vector_%s_v" % name)(ptr(dst), ptr(src0), float(src1), src0.numel(), stream_ptr()))
    return dst


class AdamState:
    """Device-side tables of one parameter list for bbhip_fp32_OptimizerAdam, with the bias-correction products kept
    on the host as the reference does (include/bb/OptimizerAdam.h:104-110, 166-180)."""

    def __init__(self, params, grads, learning_rate=0.001, beta1=0.9, beta2=0.999):
        import numpy as np
        _dev(*params, *grads)
        self.params, self.grads = list(params), list(grads)
        self.m = [torch.zeros_like(p) for p in params]
        self.v = [torch.zeros_like(p) for p in params]
        dev = params[0].device
        table = lambda ts: torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64, device=dev)
        self.t_params, self.t_grads, self.t_m, self.t_v = table(self.params), table(self.grads), table(self.m), table(self.v)
        self.t_size = torch.tensor([p.numel() for p in params], dtype=torch.int32, device=dev)
        f32 = np.float32
        self.lr, self.beta1, self.beta2 = f32(learning_rate), f32(beta1), f32(beta2)
        self.b1, self.b2 = f32(beta1), f32(beta2)

    def lr_t(self):
        import numpy as np
        one = np.float32(1.0)
        return np.float32(np.float32(self.lr * np.sqrt(one - self.b2, dtype=np.float32)) / (one - self.b1))

    def step(self):
        check(lib().bbhip_fp32_OptimizerAdam(len(self.params), ptr(self.t_size), ptr(self.t_params), ptr(self.t_grads),
                                             ptr(self.t_m), ptr(self.t_v), float(self.lr_t()), float(self.beta1),
                                             float(self.beta2), stream_ptr()))
        self.b1 = self.b1 * self.beta1
        self.b2 = self.b2 * self.beta2

    def update(self):
        """Optimizer::Update of the reference = step, then the gradients set to zero (include/bb/Optimizer.h:31-35), in one launch."""
        check(lib().bbhip_fp32_OptimizerAdam_Update(len(self.params), ptr(self.t_size), ptr(self.t_params), ptr(self.t_grads),
                                                    ptr(self.t_m), ptr(self.t_v), float(self.lr_t()), float(self.beta1),
                                                    float(self.beta2), stream_ptr()))
        self.b1 = self.b1 * self.beta1
        self.b2 = self.b2 * self.beta2


BORDER_MODES = {"constant": 0, "reflect": 1, "reflect_101": 2, "replicate": 3, "wrap": 4}


def im2col_geometry(h, w, fh, fw, ys=1, xs=1, padding="valid"):
    """(oh, ow, y_offset, x_offset) of a filter fh x fw stepping by (ys, xs) (reference: include/bb/ConvolutionIm2Col.h:183-198)"""
    if padding == "valid":
        return ((h - fh + 1) + (ys - 1)) // ys, ((w - fw + 1) + (xs - 1)) // xs, 0, 0
    if padding != "same":
        raise capi.BbhipError("padding must be 'valid' or 'same'")
    return (h + ys - 1) // ys, (w + xs - 1) // xs, (fh - 1) // 2, (fw - 1) // 2


def _stride_for(frames, bit):
    from . import synth
    return synth.frame_stride_bit(frames) if bit else synth.frame_stride_fp32(frames)


def im2col_forward(x, c, h, w, frames, fh, fw, ys=1, xs=1, padding="valid", border="reflect_101", border_value=0.0):
    """x [c*h*w, stride] float32 or packed int32 -> y [c*fh*fw, stride'] holding frames*oh*ow frames"""
    _dev(x)
    bit = x.dtype == torch.int32
    oh, ow, yo, xo = im2col_geometry(h, w, fh, fw, ys, xs, padding)
    of = frames * oh * ow
    y = (torch.zeros if bit else torch.empty)((c * fh * fw, _stride_for(of, bit)), dtype=x.dtype, device=x.device)
    if bit:
        check(lib().bbhip_bit_Im2Col_Forward(ptr(x), ptr(y), xs, ys, xo, yo, frames, x.shape[1], w, h, c, ow, oh, y.shape[1], fw, fh,
                                             BORDER_MODES[border], stream_ptr()))
    else:
        check(lib().bbhip_fp32_Im2Col_Forward(ptr(x), ptr(y), xs, ys, xo, yo, frames, x.shape[1], w, h, c, ow, oh, y.shape[1], fw, fh,
                                              BORDER_MODES[border], border_value, stream_ptr()))
    return y


def im2col_backward(dy, c, h, w, frames, fh, fw, ys=1, xs=1, padding="valid"):
    _dev(dy)
    oh, ow, yo, xo = im2col_geometry(h, w, fh, fw, ys, xs, padding)
    dx = torch.empty((c * h * w, _stride_for(frames, False)), dtype=torch.float32, device=dy.device)
    check(lib().bbhip_fp32_Im2Col_Backward(ptr(dy), ptr(dx), xs, ys, xo, yo, frames, dx.shape[1], w, h, c, ow, oh, dy.shape[1], fw, fh,
                                           stream_ptr()))
    return dx


def col2im_forward(x, c, h, w, frames):
    """x [c, stride] over frames*h*w frames -> y [c*h*w, stride'] over frames frames"""
    _dev(x)
    bit = x.dtype == torch.int32
    y = (torch.zeros if bit else torch.empty)((c * h * w, _stride_for(frames, bit)), dtype=x.dtype, device=x.device)
    fn = lib().bbhip_bit_Col2Im_Forward if bit else lib().bbhip_fp32_Col2Im_Forward
    check(fn(ptr(x), ptr(y), w, h, c, x.shape[1], frames, y.shape[1], stream_ptr()))
    return y


def col2im_backward(dy, c, h, w, frames):
    _dev(dy)
    dx = torch.empty((c, _stride_for(frames * h * w, False)), dtype=torch.float32, device=dy.device)
    check(lib().bbhip_fp32_Col2Im_Backward(ptr(dy), ptr(dx), w, h, c, dx.shape[1], frames, dy.shape[1], stream_ptr()))
    return dx


def stochastic_maxpool2x2_forward(x, c, h, w, frames):
    _dev(x)
    oh, ow = (h + 1) // 2, (w + 1) // 2
    y = torch.empty((c * oh * ow, x.shape[1]), dtype=torch.float32, device=x.device)
    check(lib().bbhip_fp32_StochasticMaxPooling2x2_Forward(ptr(x), ptr(y), w, h, ow, oh, c, frames, x.shape[1], stream_ptr()))
    return y


def stochastic_maxpool2x2_backward(x, dy, c, h, w, frames):
    _dev(x, dy)
    oh, ow = (h + 1) // 2, (w + 1) // 2
    dx = torch.empty_like(x)
    check(lib().bbhip_fp32_StochasticMaxPooling2x2_Backward(ptr(x), ptr(dy), ptr(dx), w, h, ow, oh, c, frames, x.shape[1], stream_ptr()))
    return dx


def stochastic_bn_forward_training(x, running_mean, running_var, frame_size, gamma=0.2, beta=0.5, momentum=0.9):
    """Per-node batch normalisation with scalar gamma / beta, training pass: x [nodes, stride] -> (y, mean, rstd); the running
    statistics are updated in place."""
    _dev(x, running_mean, running_var)
    nodes = x.shape[0]
    y = torch.empty_like(x)
    mean = torch.empty(nodes, dtype=torch.float32, device=x.device)
    rstd = torch.empty(nodes, dtype=torch.float32, device=x.device)
    check(lib().bbhip_fp32_StochasticBatchNormalization_ForwardTraining(ptr(x), ptr(y), ptr(mean), ptr(rstd), ptr(running_mean),
                                                                        ptr(running_var), gamma, beta, momentum, nodes, frame_size,
                                                                        x.shape[1], stream_ptr()))
    return y, mean, rstd


def stochastic_bn_reforward(x, mean, rstd, frame_size, gamma=0.2, beta=0.5):
    _dev(x, mean, rstd)
    y = torch.empty_like(x)
    check(lib().bbhip_fp32_StochasticBatchNormalization_ReForward(ptr(x), ptr(y), ptr(mean), ptr(rstd), gamma, beta, x.shape[0], frame_size,
                                                                  x.shape[1], stream_ptr()))
    return y


def stochastic_bn_forward_inference(x, running_mean, running_var, frame_size, gamma=0.2, beta=0.5):
    _dev(x, running_mean, running_var)
    y = torch.empty_like(x)
    check(lib().bbhip_fp32_StochasticBatchNormalization_ForwardInference(ptr(x), ptr(y), ptr(running_mean), ptr(running_var), gamma, beta,
                                                                         x.shape[0], frame_size, x.shape[1], stream_ptr()))
    return y


def stochastic_bn_backward(x, dy, mean, rstd, frame_size, gamma=0.2):
    _dev(x, dy, mean, rstd)
    dx = torch.empty_like(dy)
    check(lib().bbhip_fp32_StochasticBatchNormalization_Backward(ptr(x), ptr(dy), ptr(dx), ptr(mean), ptr(rstd), gamma, 1.0 / frame_size,
                                                                 dy.shape[0], frame_size, dy.shape[1], x.shape[1], stream_ptr()))
    return dx


def average_lut_forward(x, idx, frame_size, binarize_input=False, binarize_output=True, mean=True):
    """fp32 x [I, stride] -> y [O, stride]: the sign of the sum of the n wired inputs (their votes when binarize_input) or, without
    binarize_output, sum * (1 / n) as the reference's CUDA kernel writes it; mean=False: the plain sum of the reference's host loop."""
    _dev(x, idx)
    O, n = idx.shape
    y = torch.empty((O, x.shape[1]), dtype=torch.float32, device=x.device)
    entry = lib().bbhip_fp32_AverageLut_Forward if mean else lib().bbhip_fp32_AverageLut_ForwardSum
    check(entry(ptr(x), ptr(y), ptr(idx), n, O, frame_size, x.shape[1], int(binarize_input), int(binarize_output), stream_ptr()))
    return y


def bit_average_lut_forward(xbits, idx, frame_size):
    """packed x [I, words] -> packed y [O, words]: strict majority of the n wired inputs."""
    _dev(xbits, idx)
    O, n = idx.shape
    y = torch.zeros((O, xbits.shape[1]), dtype=torch.int32, device=xbits.device)
    check(lib().bbhip_bit_AverageLut_Forward(ptr(xbits), ptr(y), ptr(idx), n, O, frame_size, xbits.shape[1], stream_ptr()))
    return y


def average_lut_backward(dy, idx, input_nodes, frame_size):
    _dev(dy, idx)
    O, n = idx.shape
    dx = torch.empty((input_nodes, dy.shape[1]), dtype=torch.float32, device=dy.device)
    check(lib().bbhip_fp32_AverageLut_Backward(ptr(dy), ptr(dx), ptr(idx), n, input_nodes, O, frame_size, dy.shape[1], stream_ptr()))
    return dx


def max_lut_forward(x, idx, frame_size, binarize_input=False, binarize_output=True):
    """fp32 x [I, stride] -> y [O, stride]: the largest of the n wired inputs (not below -1), or its sign."""
    _dev(x, idx)
    O, n = idx.shape
    y = torch.empty((O, x.shape[1]), dtype=torch.float32, device=x.device)
    check(lib().bbhip_fp32_MaxLut_Forward(ptr(x), ptr(y), ptr(idx), n, O, frame_size, x.shape[1], int(binarize_input), int(binarize_output),
                                          stream_ptr()))
    return y


def bit_max_lut_forward(xbits, idx, frame_size):
    """packed x [I, words] -> packed y [O, words]: the OR of the n wired inputs."""
    _dev(xbits, idx)
    O, n = idx.shape
    y = torch.empty((O, xbits.shape[1]), dtype=torch.int32, device=xbits.device)
    check(lib().bbhip_bit_MaxLut_Forward(ptr(xbits), ptr(y), ptr(idx), n, O, frame_size, xbits.shape[1], stream_ptr()))
    return y


def max_lut_backward(x, dy, idx, frame_size, binarize_input=False):
    """dx [I, stride]: each node's dy goes to its first largest input."""
    _dev(x, dy, idx)
    O, n = idx.shape
    if x.shape[1] != dy.shape[1]:
        raise capi.BbhipError("max_lut_backward: x and dy must have the same row pitch")
    dx = torch.empty((x.shape[0], dy.shape[1]), dtype=torch.float32, device=dy.device)
    check(lib().bbhip_fp32_MaxLut_Backward(ptr(x), ptr(dy), ptr(dx), ptr(idx), n, x.shape[0], O, frame_size, dy.shape[1], int(binarize_input),
                                           stream_ptr()))
    return dx


def bit_max_lut_backward(xbits, dy, idx, frame_size):
    _dev(xbits, dy, idx)
    O, n = idx.shape
    dx = torch.empty((xbits.shape[0], dy.shape[1]), dtype=torch.float32, device=dy.device)
    check(lib().bbhip_bit_fp32_MaxLut_Backward(ptr(xbits), ptr(dy), ptr(dx), ptr(idx), n, xbits.shape[0], O, frame_size, xbits.shape[1],
                                               dy.shape[1], stream_ptr()))
    return dx


def reduce_forward(x, output_nodes, frame_size):
    """fp32 x [I, stride] -> y [O, stride]: node o is the mean of the inputs o, O + o, 2 O + o, ..."""
    _dev(x)
    y = torch.empty((output_nodes, x.shape[1]), dtype=torch.float32, device=x.device)
    check(lib().bbhip_fp32_Reduce_Forward(ptr(x), ptr(y), x.shape[0], output_nodes, frame_size, x.shape[1], stream_ptr()))
    return y


def bit_reduce_forward(xbits, output_nodes, frame_size, y_stride):
    """packed x [I, words] (bits read as +1 / -1) -> fp32 y [O, y_stride]"""
    _dev(xbits)
    y = torch.empty((output_nodes, y_stride), dtype=torch.float32, device=xbits.device)
    check(lib().bbhip_bit_fp32_Reduce_Forward(ptr(xbits), ptr(y), xbits.shape[0], output_nodes, frame_size, xbits.shape[1], y_stride, stream_ptr()))
    return y


def reduce_backward(dy, input_nodes, frame_size):
    _dev(dy)
    dx = torch.empty((input_nodes, dy.shape[1]), dtype=torch.float32, device=dy.device)
    check(lib().bbhip_fp32_Reduce_Backward(ptr(dy), ptr(dx), input_nodes, dy.shape[0], frame_size, dy.shape[1], stream_ptr()))
    return dx


def real_to_binary_forward(x, depth, points, frame_size, frame_mod=1, depth_mod=1, lo=0.0, hi=1.0, binarize=True, bit=False, y_stride=None):
    """fp32 x [depth * points, stride] -> y [depth * depth_mod * points, y_stride]: fp32, or rows of packed words with `bit`
    (padding words of a packed row beyond the last frame's word are left as allocated: zero)."""
    _dev(x)
    out_frames = frame_size * frame_mod
    if y_stride is None:
        y_stride = (out_frames + 31) // 32 if bit else out_frames
    nodes = depth * depth_mod * points
    if bit:
        y = torch.zeros((nodes, y_stride), dtype=torch.int32, device=x.device)
        f = lib().bbhip_fp32_bit_RealToBinary_Forward
    else:
        y = torch.empty((nodes, y_stride), dtype=torch.float32, device=x.device)
        f = lib().bbhip_fp32_RealToBinary_Forward
    check(f(ptr(x), ptr(y), depth_mod, frame_mod, lo, hi, points, depth, frame_size, x.shape[1], y_stride, int(binarize), stream_ptr()))
    return y


def binary_to_real_forward(x, output_nodes, y_frame_size, frame_mux=1, y_stride=None):
    """x [I, stride] fp32 (counted where > 0) or int32 packed bits, y_frame_size * frame_mux frames -> fp32 y [O, y_stride]"""
    _dev(x)
    y_stride = y_frame_size if y_stride is None else y_stride
    y = torch.empty((output_nodes, y_stride), dtype=torch.float32, device=x.device)
    f = lib().bbhip_bit_fp32_BinaryToReal_Forward if x.dtype == torch.int32 else lib().bbhip_fp32_BinaryToReal_Forward
    check(f(ptr(x), ptr(y), x.shape[0] // output_nodes, frame_mux, output_nodes, x.shape[1], y_frame_size, y_stride, stream_ptr()))
    return y


def binary_to_real_backward(dy, input_nodes, y_frame_size, frame_mux=1, x_stride=None):
    _dev(dy)
    x_stride = y_frame_size * frame_mux if x_stride is None else x_stride
    dx = torch.empty((input_nodes, x_stride), dtype=torch.float32, device=dy.device)
    check(lib().bbhip_fp32_BinaryToReal_Backward(ptr(dy), ptr(dx), input_nodes // dy.shape[0], frame_mux, dy.shape[0], x_stride, y_frame_size,
                                                 dy.shape[1], stream_ptr()))
    return dx


def binarize_forward(x, frame_size, th=0.0, low=-1.0, high=1.0, bit=False, y_stride=None):
    """y = x > th ? high : low, or with `bit` the packed bits of x > th"""
    _dev(x)
    if bit:
        y_stride = (frame_size + 31) // 32 if y_stride is None else y_stride
        y = torch.zeros((x.shape[0], y_stride), dtype=torch.int32, device=x.device)
        check(lib().bbhip_fp32_bit_Binarize_Forward(ptr(x), ptr(y), th, x.shape[0], frame_size, x.shape[1], y_stride, stream_ptr()))
        return y
    y = torch.empty_like(x)
    check(lib().bbhip_fp32_Binarize_Forward(ptr(x), ptr(y), th, low, high, x.shape[0], frame_size, x.shape[1], stream_ptr()))
    return y


def hard_tanh_forward(x, frame_size, lo=-1.0, hi=1.0):
    _dev(x)
    y = torch.empty_like(x)
    check(lib().bbhip_fp32_HardTanh_Forward(ptr(x), ptr(y), lo, hi, x.shape[0], frame_size, x.shape[1], stream_ptr()))
    return y


def hard_tanh_backward(x, dy, frame_size, lo=-1.0, hi=1.0):
    """dx = dy inside the open window (lo, hi), 0 elsewhere; also the backward of Binarize"""
    _dev(x, dy)
    dx = torch.empty_like(dy)
    check(lib().bbhip_fp32_HardTanh_Backward(ptr(x), ptr(dy), ptr(dx), lo, hi, x.shape[0], frame_size, x.shape[1], stream_ptr()))
    return dx


def _pool_out(h, w, fh, fw):
    return (h + fh - 1) // fh, (w + fw - 1) // fw


def max_pooling_forward(x, c, h, w, fh, fw, frame_size):
    """fp32 x [c * h * w, stride] -> (y, argmax) [c * oh * ow, stride]"""
    _dev(x)
    oh, ow = _pool_out(h, w, fh, fw)
    y = torch.empty((c * oh * ow, x.shape[1]), dtype=torch.float32, device=x.device)
    arg = torch.empty((c * oh * ow, x.shape[1]), dtype=torch.int32, device=x.device)
    check(lib().bbhip_fp32_MaxPooling_Forward(ptr(x), ptr(y), ptr(arg), fh, fw, w, h, ow, oh, c, frame_size, x.shape[1], stream_ptr()))
    return y, arg


def max_pooling_backward(argmax, dy, c, h, w, fh, fw, frame_size):
    _dev(argmax, dy)
    oh, ow = _pool_out(h, w, fh, fw)
    dx = torch.empty((c * h * w, dy.shape[1]), dtype=torch.float32, device=dy.device)
    check(lib().bbhip_fp32_MaxPooling_Backward(ptr(argmax), ptr(dy), ptr(dx), fh, fw, w, h, ow, oh, c, frame_size, dy.shape[1], stream_ptr()))
    return dx


def bit_max_pooling_forward(xbits, c, h, w, fh, fw, frame_size):
    _dev(xbits)
    oh, ow = _pool_out(h, w, fh, fw)
    y = torch.zeros((c * oh * ow, xbits.shape[1]), dtype=torch.int32, device=xbits.device)
    check(lib().bbhip_bit_MaxPooling_Forward(ptr(xbits), ptr(y), fh, fw, w, h, ow, oh, c, frame_size, xbits.shape[1], stream_ptr()))
    return y


def bit_max_pooling_backward(xbits, dy, c, h, w, fh, fw, frame_size):
    _dev(xbits, dy)
    oh, ow = _pool_out(h, w, fh, fw)
    dx = torch.empty((c * h * w, dy.shape[1]), dtype=torch.float32, device=dy.device)
    check(lib().bbhip_bit_fp32_MaxPooling_Backward(ptr(xbits), ptr(dy), ptr(dx), fh, fw, w, h, ow, oh, c, frame_size, xbits.shape[1], dy.shape[1],
                                                   stream_ptr()))
    return dx


def up_sampling_forward(x, c, h, w, fh, fw, frame_size, fill=True):
    """x [c * h * w, stride], fp32 or int32 packed words -> y [c * h fh * w fw, stride] of the same type"""
    _dev(x)
    if x.dtype == torch.int32:
        y = torch.zeros((c * h * fh * w * fw, x.shape[1]), dtype=torch.int32, device=x.device)
        f = lib().bbhip_bit_UpSampling_Forward
    else:
        y = torch.empty((c * h * fh * w * fw, x.shape[1]), dtype=torch.float32, device=x.device)
        f = lib().bbhip_fp32_UpSampling_Forward
    check(f(ptr(x), ptr(y), w, h, c, fw, fh, int(fill), frame_size, x.shape[1], stream_ptr()))
    return y


def up_sampling_backward(dy, c, h, w, fh, fw, frame_size, fill=True):
    _dev(dy)
    dx = torch.empty((c * h * w, dy.shape[1]), dtype=torch.float32, device=dy.device)
    check(lib().bbhip_fp32_UpSampling_Backward(ptr(dy), ptr(dx), w, h, c, fw, fh, int(fill), frame_size, dy.shape[1], stream_ptr()))
    return dx


def shuffle_forward(x, shuffle_unit, frame_size):
    """x [nodes, stride], fp32 or int32 packed words: row i * shuffle_unit + j of the result is row j * (nodes / shuffle_unit) + i"""
    _dev(x)
    y = torch.empty_like(x)
    check(lib().bbhip_Shuffle_Forward(ptr(x), ptr(y), shuffle_unit, x.shape[0], frame_size, x.shape[1], stream_ptr()))
    return y


def shuffle_backward(dy, shuffle_unit, frame_size):
    _dev(dy)
    dx = torch.empty_like(dy)
    check(lib().bbhip_Shuffle_Backward(ptr(dy), ptr(dx), shuffle_unit, dy.shape[0], frame_size, dy.shape[1], stream_ptr()))
    return dx


def loss_mean_squared_error(y, t, frame_size, loss_buf, batch_size=None, reduction_sum=False):
    """-> dy; loss_buf (float64, device, any length >= 1) receives the batch's partial sums ON TOP of what it holds.  The layer's loss is
    loss_buf.sum() / frames seen (the sum itself with reduction "sum")."""
    _dev(y, t, loss_buf)
    nodes = y.shape[0]
    batch_size = frame_size if batch_size is None else batch_size
    import numpy as np
    grad_reduction = np.float32(1.0) if reduction_sum else np.float32(1.0) / np.float32(nodes * batch_size)
    loss_reduction = 1.0 if reduction_sum else 1.0 / nodes
    dy = torch.empty_like(y)
    check(lib().bbhip_fp32_LossMeanSquaredError(ptr(y), ptr(t), ptr(dy), ptr(loss_buf), loss_buf.numel(), nodes, frame_size, y.shape[1],
                                                float(np.float32(2) * grad_reduction), loss_reduction, stream_ptr()))
    return dy


def metrics_mean_squared_error(y, t, frame_size, accuracy_buf):
    """accuracy_buf (float64, device) += the batch's partial sums of (t - y)^2 / nodes; the metric is accuracy_buf.sum() / frames seen."""
    _dev(y, t, accuracy_buf)
    check(lib().bbhip_fp32_MetricsMeanSquaredError(ptr(y), ptr(t), ptr(accuracy_buf), accuracy_buf.numel(), y.shape[0], frame_size, y.shape[1],
                                                   stream_ptr()))


def loss_softmax_cross_entropy(y, t, ch_size, pix_size, frame_size, t_sum=None):
    """y, t [ch*pix, stride] -> (dy, loss_buf [frames] float64, t_sum).  t_sum defaults to the sum of the targets of the
    frames in use, taken in float64 as the reference's device path does; the loss of the batch is -loss_buf.sum() / t_sum."""
    _dev(y, t)
    if t_sum is None:
        t_sum = float(t[:, :frame_size].sum(dtype=torch.float64).item())
    dy = torch.empty_like(y)
    loss_buf = torch.empty((frame_size,), dtype=torch.float64, device=y.device)
    check(lib().bbhip_fp32_LossSoftmaxCrossEntropy(ptr(y), ptr(t), ptr(dy), ptr(loss_buf), t_sum, pix_size, ch_size, frame_size, y.shape[1],
                                                   stream_ptr()))
    return dy, loss_buf, t_sum


def metrics_categorical_accuracy(y, t, ch_size, pix_size, frame_size):
    """-> (accuracy_buf, category_buf) int32 [frames]; the metric of the batch is the ratio of their sums."""
    _dev(y, t)
    acc = torch.empty((frame_size,), dtype=torch.int32, device=y.device)
    cat = torch.empty((frame_size,), dtype=torch.int32, device=y.device)
    check(lib().bbhip_fp32_MetricsCategoricalAccuracy(ptr(y), ptr(t), ptr(acc), ptr(cat), pix_size, ch_size, frame_size, y.shape[1], stream_ptr()))
    return acc, cat


def classifier_tail(x, idx, t, frame_size, t_sum=None, binarize_input=False, mean=True, want_y=True, want_dy=False, want_accuracy=True):
    """AverageLut forward (un-binarized) + softmax cross entropy + categorical accuracy + AverageLut backward in one launch; the same
    bits as `average_lut_forward`, `loss_softmax_cross_entropy`, `metrics_categorical_accuracy` and `average_lut_backward` called one
    after the other.  returns (y or None, dx, loss_buf, accuracy or None, category or None, dy or None)."""
    _dev(x, idx, t)
    ch, n = idx.shape
    S = x.shape[1]
    assert t.shape[1] == S
    y = torch.empty((ch, S), dtype=torch.float32, device=x.device) if want_y else None
    dy = torch.empty((ch, S), dtype=torch.float32, device=x.device) if want_dy else None
    dx = torch.empty((x.shape[0], S), dtype=torch.float32, device=x.device)
    loss_buf = torch.empty(frame_size, dtype=torch.float64, device=x.device)
    acc = torch.empty(frame_size, dtype=torch.int32, device=x.device) if want_accuracy else None
    cat = torch.empty(frame_size, dtype=torch.int32, device=x.device) if want_accuracy else None
    if t_sum is None:
        t_sum = float(t[:, :frame_size].sum(dtype=torch.float64).item())
    check(lib().bbhip_fp32_ClassifierTail_ForwardBackward(ptr(x), ptr(y), ptr(dx), ptr(idx), ptr(t), ptr(dy), ptr(loss_buf), ptr(acc), ptr(cat),
                                                          float(t_sum), n, x.shape[0], ch, frame_size, S,
                                                          int(binarize_input), int(not mean), stream_ptr()))
    return y, dx, loss_buf, acc, cat, dy


def conv_bit_to_real(xbits, frame_size, y_stride, value0=0.0, value1=1.0):
    _dev(xbits)
    y = torch.empty((xbits.shape[0], y_stride), dtype=torch.float32, device=xbits.device)
    check(lib().bbhip_fp32_ConvBitToReal(ptr(xbits), ptr(y), value0, value1, xbits.shape[0], frame_size,
                                         xbits.shape[1], y_stride, stream_ptr()))
    return y


def packed_input_buffer(rows, frame_size, device="cuda"):
    """A place for the packed copy of a binarized fp32 input of `rows` node rows (see `packed=` of the LUT forward / backward wrappers):
    the forward call fills it, the backward call on the same input reads it instead of packing the input again."""
    return torch.empty((rows, lib().bbhip_PackedRowWords(frame_size)), dtype=torch.int32, device=device)


def prepared_tables_buffer(n, node_size, device="cuda"):
    """A buffer for bbhip_HintPreparedTables: the tables that a LUT call derives from W, kept from a step's forward call for its
    backward call (`tables=` of the DifferentiableLut wrappers)."""
    return torch.empty(lib().bbhip_PreparedTablesBytes(n, node_size) // 4, dtype=torch.float32, device=device)


def _hint_tables(tables, holds_tables):
    if tables is not None and HINTS:
        _dev(tables)
        assert tables.dtype == torch.float32
        lib().bbhip_HintPreparedTables(ptr(tables), tables.numel() * 4, int(holds_tables))


HINTS = True          # False: the wrappers pass no bbhip_Hint* at all (what a caller of the reference's plain signatures gets)


def _hint_input(x, packed, holds_input, forward=True):
    """what the wrapper knows about the next LUT call's input: its row count, and where its packed copy goes to / comes from"""
    if not HINTS:
        return
    if packed is not None:
        _dev(packed)
        assert packed.dtype == torch.int32 and packed.shape[0] == x.shape[0]
        lib().bbhip_HintPackedInput(ptr(packed), x.shape[0], packed.shape[1], int(holds_input))
    elif forward:
        lib().bbhip_HintInputNodeSize(x.shape[0])       # the forward signatures do not carry the row count of x


def _hint_output(packed_out, rows):
    """packed_out: a `packed_input_buffer(rows, frame_size)` that receives the binarized output as packed bits (for the next layer)"""
    if packed_out is not None and HINTS:
        _dev(packed_out)
        assert packed_out.dtype == torch.int32 and packed_out.shape[0] == rows
        lib().bbhip_HintPackedOutput(ptr(packed_out), rows, packed_out.shape[1])


def _hint_overwrite(overwrite_dw):
    if overwrite_dw:
        lib().bbhip_HintTableGradientOverwrite(1)


def stochastic_lut_forward(n, x, idx, W, frame_size, input_binary=False, lut_binarize=False, bias=0.25, out=None, clamp_w=None, packed=None,
                           packed_holds=False):
    """clamp_w = (lo, hi): W is clamped in place first, as StochasticLutN::Forward does (include/bb/StochasticLutN.h:451),
    by the same launch that prepares the tables."""
    _dev(x, idx, W, out)
    O = idx.shape[0]
    y = torch.empty((O, x.shape[1]), dtype=torch.float32, device=x.device) if out is None else out
    _hint_input(x, packed, packed_holds)
    if clamp_w is not None:
        check(lib().bbhip_fp32_StochasticLut_ForwardClampW(n, ptr(x), ptr(y), ptr(idx), ptr(W), O, frame_size, x.shape[1],
                                                           int(input_binary), int(lut_binarize), bias, float(clamp_w[0]), float(clamp_w[1]), stream_ptr()))
        return y
    check(lib().bbhip_fp32_StochasticLut_Forward(n, ptr(x), ptr(y), ptr(idx), ptr(W), O, frame_size, x.shape[1],
                                                 int(input_binary), int(lut_binarize), bias, stream_ptr()))
    return y


def bit_stochastic_lut_forward(n, xbits, idx, W, frame_size, y_stride, lut_binarize=False, bias=0.25):
    _dev(xbits, idx, W)
    O = idx.shape[0]
    y = torch.empty((O, y_stride), dtype=torch.float32, device=xbits.device)
    check(lib().bbhip_bit_fp32_StochasticLut_Forward(n, ptr(xbits), ptr(y), ptr(idx), ptr(W), O, frame_size, y_stride,
                                                     xbits.shape[1], int(lut_binarize), bias, stream_ptr()))
    return y


def bit_bit_stochastic_lut_forward(n, xbits, idx, W, frame_size, lut_binarize=False, bias=0.25):
    _dev(xbits, idx, W)
    O = idx.shape[0]
    y = torch.zeros((O, xbits.shape[1]), dtype=torch.int32, device=xbits.device)
    check(lib().bbhip_bit_bit_fp32_StochasticLut_Forward(n, ptr(xbits), ptr(y), ptr(idx), ptr(W), O, frame_size,
                                                         xbits.shape[1], int(lut_binarize), bias, stream_ptr()))
    return y


def _tmp_frames(output_nodes, n, frame_size, max_tmp_bytes=256 * 1024 * 1024):
    """Frames per dx_tmp pass, as the reference sizes its scratch (include/bb/StochasticLutN.h:584-587)."""
    t = max_tmp_bytes // (4 * output_nodes * n)
    t = max(t, 32)
    t = (t + 31) & ~0x1f
    return min(t, frame_size)


def _tmp_for(output_nodes, n, frame_size, device, max_tmp_bytes):
    tf = _tmp_frames(output_nodes, n, frame_size, max_tmp_bytes)
    ts = ((tf + 63) // 64) * 64
    return torch.empty((output_nodes * n, ts), dtype=torch.float32, device=device), tf, ts


def stochastic_lut_backward(n, x, dy, idx, W, dW, frame_size, rev=None, input_binary=False, lut_binarize=False, bias=0.25,
                            dx_tmp=None, tmp_frame_size=None, max_tmp_bytes=256 * 1024 * 1024, out=None, packed=None, overwrite_dw=False):
    """dW is accumulated in place; returns dx [I, stride]. ``rev`` (reverse table) is needed by dx modes 0 and 2,
    dx_tmp by mode 2 only (allocated here when not given)."""
    _dev(x, dy, idx, W, dW, rev, dx_tmp, out)
    I = x.shape[0]; O = idx.shape[0]
    dx = torch.empty((I, dy.shape[1]), dtype=torch.float32, device=x.device) if out is None else out
    tf = ts = 0
    if dx_tmp is not None:                      # always described to the library: mode 2 needs it, mode 0 may fall back to it
        ts = dx_tmp.shape[1]
        tf = min(ts, frame_size) if tmp_frame_size is None else tmp_frame_size
    elif lib().bbhip_GetDxMode() == 2:
        dx_tmp, tf, ts = _tmp_for(O, n, frame_size, x.device, max_tmp_bytes)
    _hint_input(x, packed, True, forward=False)
    _hint_overwrite(overwrite_dw)
    check(lib().bbhip_fp32_StochasticLut_Backward(n, ptr(x), ptr(dy), ptr(dx), ptr(dx_tmp), ptr(idx), ptr(rev), ptr(W), ptr(dW),
                                                  0 if rev is None else rev.shape[1], I, O, frame_size, dy.shape[1], tf, ts,
                                                  int(input_binary), int(lut_binarize), bias, stream_ptr()))
    return dx


def bit_stochastic_lut_backward(n, xbits, dy, idx, W, dW, frame_size, rev=None, lut_binarize=False, bias=0.25,
                                max_tmp_bytes=256 * 1024 * 1024):
    _dev(xbits, dy, idx, W, dW, rev)
    I = xbits.shape[0]; O = idx.shape[0]
    dx = torch.empty((I, dy.shape[1]), dtype=torch.float32, device=dy.device)
    dx_tmp, tf, ts = (None, 0, 0)
    if lib().bbhip_GetDxMode() == 2:
        dx_tmp, tf, ts = _tmp_for(O, n, frame_size, dy.device, max_tmp_bytes)
    check(lib().bbhip_bit_fp32_StochasticLut_Backward(n, ptr(xbits), ptr(dy), ptr(dx), ptr(dx_tmp), ptr(idx), ptr(rev), ptr(W), ptr(dW),
                                                      0 if rev is None else rev.shape[1], I, O, frame_size, dy.shape[1],
                                                      xbits.shape[1], tf, ts, int(lut_binarize), bias, stream_ptr()))
    return dx


def differentiable_lut_forward_training(n, x, idx, W, frame_size, running_mean, running_var, gamma=0.3, beta=0.5,
                                        momentum=0.9, bias=0.25, lut_binarize=False, binary_mode=True, clamp_w=None, packed=None, tables=None,
                                        packed_holds=False, packed_out=None):
    """fp32 frames. running_mean / running_var are updated in place. returns (y, mean, rstd).
    packed_holds: `packed` already holds the packed copy of x (it was the `packed_out` of the layer before): nothing is packed.
    packed_out: a `packed_input_buffer(O, frame_size)` that receives the binarized output as packed bits, for the next layer.
    tables: a `prepared_tables_buffer` that receives the tables derived from W, for the backward call of the same step.
    packed: a `packed_input_buffer` that receives the packed copy of the binarized input (binary mode), for the backward call.
    clamp_w = (lo, hi): W is clamped in place first, by the launch that prepares the tables (the model class's clamp before the
    first forward pass after a backward pass, include/bb/DifferentiableLutN.h:605-608)."""
    _dev(x, idx, W, running_mean, running_var)
    O = idx.shape[0]
    y = torch.empty((O, x.shape[1]), dtype=torch.float32, device=x.device)
    mean = torch.empty(O, dtype=torch.float32, device=x.device)
    rstd = torch.empty(O, dtype=torch.float32, device=x.device)
    _hint_input(x, packed, packed_holds)
    _hint_tables(tables, False)
    _hint_output(packed_out if binary_mode else None, O)
    if clamp_w is not None:
        check(lib().bbhip_fp32_DifferentiableLutN_ForwardTrainingClampW(n, ptr(x), ptr(y), ptr(idx), ptr(W), ptr(mean), ptr(rstd),
                                                                        ptr(running_mean), ptr(running_var), gamma, beta, momentum, bias,
                                                                        O, frame_size, x.shape[1], int(lut_binarize), int(binary_mode),
                                                                        float(clamp_w[0]), float(clamp_w[1]), stream_ptr()))
        return y, mean, rstd
    check(lib().bbhip_fp32_DifferentiableLutN_ForwardTraining(n, ptr(x), ptr(y), ptr(idx), ptr(W), ptr(mean), ptr(rstd),
                                                              ptr(running_mean), ptr(running_var), gamma, beta, momentum, bias,
                                                              O, frame_size, x.shape[1], int(lut_binarize), int(binary_mode),
                                                              stream_ptr()))
    return y, mean, rstd


def bit_differentiable_lut_forward_training(n, xbits, idx, W, frame_size, running_mean, running_var, gamma=0.3, beta=0.5,
                                            momentum=0.9, bias=0.25, lut_binarize=False, clamp_w=None, tables=None, out=None):
    """out: a packed output buffer [O, words] to write into (a layer keeps one); None: a new zero-filled one."""
    _dev(xbits, idx, W, running_mean, running_var)
    O = idx.shape[0]
    y = out if out is not None else torch.zeros((O, xbits.shape[1]), dtype=torch.int32, device=xbits.device)
    if tuple(y.shape) != (O, xbits.shape[1]) or y.dtype != torch.int32:
        raise ValueError("out must be int32 [%d, %d]" % (O, xbits.shape[1]))
    mean = torch.empty(O, dtype=torch.float32, device=xbits.device)
    rstd = torch.empty(O, dtype=torch.float32, device=xbits.device)
    _hint_tables(tables, False)
    if clamp_w is not None:
        check(lib().bbhip_bit_fp32_DifferentiableLutN_ForwardTrainingClampW(n, ptr(xbits), ptr(y), ptr(idx), ptr(W), ptr(mean), ptr(rstd),
                                                                            ptr(running_mean), ptr(running_var), gamma, beta, momentum, bias,
                                                                            O, frame_size, xbits.shape[1], int(lut_binarize),
                                                                            float(clamp_w[0]), float(clamp_w[1]), stream_ptr()))
        return y, mean, rstd
    check(lib().bbhip_bit_fp32_DifferentiableLutN_ForwardTraining(n, ptr(xbits), ptr(y), ptr(idx), ptr(W), ptr(mean), ptr(rstd),
                                                                  ptr(running_mean), ptr(running_var), gamma, beta, momentum, bias,
                                                                  O, frame_size, xbits.shape[1], int(lut_binarize), stream_ptr()))
    return y, mean, rstd


def differentiable_lut_forward_inference(n, x, idx, W, frame_size, running_mean, running_var, gamma=0.3, beta=0.5,
                                         bias=0.25, lut_binarize=False, binary_mode=True, packed=None, packed_holds=False, packed_out=None):
    _dev(x, idx, W, running_mean, running_var)
    O = idx.shape[0]
    y = torch.empty((O, x.shape[1]), dtype=torch.float32, device=x.device)
    _hint_input(x, packed, packed_holds)
    _hint_output(packed_out if binary_mode else None, O)
    check(lib().bbhip_fp32_DifferentiableLutN_ForwardInference(n, ptr(x), ptr(y), ptr(idx), ptr(W), ptr(running_mean),
                                                               ptr(running_var), gamma, beta, bias, O, frame_size, x.shape[1],
                                                               int(lut_binarize), int(binary_mode), stream_ptr()))
    return y


def bit_differentiable_lut_forward_inference(n, xbits, idx, W, frame_size, running_mean, running_var, gamma=0.3,
                                             beta=0.5, bias=0.25, lut_binarize=False):
    _dev(xbits, idx, W, running_mean, running_var)
    O = idx.shape[0]
    y = torch.zeros((O, xbits.shape[1]), dtype=torch.int32, device=xbits.device)
    check(lib().bbhip_bit_fp32_DifferentiableLutN_ForwardInference(n, ptr(xbits), ptr(y), ptr(idx), ptr(W), ptr(running_mean),
                                                                   ptr(running_var), gamma, beta, bias, O, frame_size,
                                                                   xbits.shape[1], int(lut_binarize), stream_ptr()))
    return y


def differentiable_lut_forward_nobn(n, x, idx, W, frame_size, bias=0.25, lut_binarize=False, binary_mode=True, packed=None, packed_holds=False,
                                    packed_out=None):
    _dev(x, idx, W)
    O = idx.shape[0]
    y = torch.empty((O, x.shape[1]), dtype=torch.float32, device=x.device)
    _hint_input(x, packed, packed_holds)
    _hint_output(packed_out if binary_mode else None, O)
    check(lib().bbhip_fp32_DifferentiableLutN_ForwardNoBn(n, ptr(x), ptr(y), ptr(idx), ptr(W), bias, O, frame_size, x.shape[1],
                                                          int(lut_binarize), int(binary_mode), stream_ptr()))
    return y


def differentiable_lut_backward(n, x, dy, idx, W, dW, frame_size, mean, rstd, rev=None, gamma=0.3, beta=0.5, bias=0.25,
                                lut_binarize=False, binary_mode=True, max_tmp_bytes=256 * 1024 * 1024, packed=None, tables=None, overwrite_dw=False):
    """tables: the buffer that this step's forward call with the same W filled (`prepared_tables_buffer`): no preparation launch.
    packed: the buffer that the forward call on the same x filled (`packed_input_buffer`): the call reads it instead of packing x."""
    _dev(x, dy, idx, W, dW, mean, rstd, rev)
    I = x.shape[0]; O = idx.shape[0]
    dx = torch.empty((I, dy.shape[1]), dtype=torch.float32, device=x.device)
    dmean = torch.empty(O, dtype=torch.float32, device=x.device)
    dvar = torch.empty(O, dtype=torch.float32, device=x.device)
    dx_tmp, tf, ts = (None, 0, 0)
    if lib().bbhip_GetDxMode() == 2:
        dx_tmp, tf, ts = _tmp_for(O, n, frame_size, x.device, max_tmp_bytes)
    _hint_input(x, packed, True, forward=False)
    _hint_tables(tables, True)
    _hint_overwrite(overwrite_dw)
    check(lib().bbhip_fp32_DifferentiableLutN_Backward(n, ptr(x), ptr(dy), ptr(dx), ptr(dx_tmp), ptr(idx), ptr(rev), ptr(W), ptr(dW),
                                                       ptr(mean), ptr(rstd), ptr(dmean), ptr(dvar), gamma, beta, bias,
                                                       0 if rev is None else rev.shape[1], I, O, frame_size, dy.shape[1], tf, ts,
                                                       int(lut_binarize), int(binary_mode), stream_ptr()))
    return dx


def bit_differentiable_lut_backward(n, xbits, dy, idx, W, dW, frame_size, mean, rstd, rev=None, gamma=0.3, beta=0.5,
                                    bias=0.25, lut_binarize=False, max_tmp_bytes=256 * 1024 * 1024, tables=None):
    _dev(xbits, dy, idx, W, dW, mean, rstd, rev)
    I = xbits.shape[0]; O = idx.shape[0]
    dx = torch.empty((I, dy.shape[1]), dtype=torch.float32, device=dy.device)
    dmean = torch.empty(O, dtype=torch.float32, device=dy.device)
    dvar = torch.empty(O, dtype=torch.float32, device=dy.device)
    dx_tmp, tf, ts = (None, 0, 0)
    if lib().bbhip_GetDxMode() == 2:
        dx_tmp, tf, ts = _tmp_for(O, n, frame_size, dy.device, max_tmp_bytes)
    _hint_tables(tables, True)
    check(lib().bbhip_bit_fp32_DifferentiableLutN_Backward(n, ptr(xbits), ptr(dy), ptr(dx), ptr(dx_tmp), ptr(idx), ptr(rev), ptr(W),
                                                           ptr(dW), ptr(mean), ptr(rstd), ptr(dmean), ptr(dvar), gamma, beta, bias,
                                                           0 if rev is None else rev.shape[1], I, O, frame_size, dy.shape[1],
                                                           xbits.shape[1], tf, ts, int(lut_binarize), stream_ptr()))
    return dx


def binary_lut6_forward(xbits, idx, table, frame_size, out=None):
    _dev(xbits, idx, table, out)
    O = idx.shape[0]
    y = torch.zeros((O, xbits.shape[1]), dtype=torch.int32, device=xbits.device) if out is None else out
    check(lib().bbhip_bit_BinaryLut6_Forward(ptr(xbits), ptr(y), ptr(idx), ptr(table), O, frame_size, xbits.shape[1], stream_ptr()))
    return y


def binary_lutn_forward(n, xbits, idx, table, frame_size, out=None):
    """BinaryLutN<n> on packed bits, n = 2 .. 6: table [O, 1] words for n <= 5 (entry i = bit i), [O, 2] for n = 6"""
    _dev(xbits, idx, table, out)
    O = idx.shape[0]
    assert idx.shape[1] == n and table.shape == (O, 2 if n == 6 else 1)
    y = torch.zeros((O, xbits.shape[1]), dtype=torch.int32, device=xbits.device) if out is None else out
    check(lib().bbhip_bit_BinaryLutN_Forward(n, ptr(xbits), ptr(y), ptr(idx), ptr(table), O, frame_size, xbits.shape[1], stream_ptr()))
    return y


def reverse_table(idx, input_nodes):
    """Reverse connection table as the reference builds it (include/bb/FixedSizeConnectionTable.h:180-215):
    ``[input_nodes, 1 + max fan-out]`` int32, row r = [count, node*n + input ... ascending, zero tail].
    Built on the host with numpy (index bookkeeping, not on the timed path); returned on idx's device."""
    import numpy as np
    h = idx.detach().cpu().numpy().astype(np.int64)
    O, n = h.shape
    flat = h.reshape(-1)
    counts = np.bincount(flat, minlength=input_nodes)
    stride = int(counts.max()) + 1 if flat.size else 1
    order = np.argsort(flat, kind="stable")                      # ascending (node, input) within each input row
    starts = np.concatenate([[0], np.cumsum(counts)[:-1]])
    rev = np.zeros((input_nodes, stride), np.int32)
    rev[:, 0] = counts
    pos = np.arange(flat.size) - np.repeat(starts, counts)
    rev[flat[order], 1 + pos] = order.astype(np.int32)
    return torch.from_numpy(rev).to(idx.device)
