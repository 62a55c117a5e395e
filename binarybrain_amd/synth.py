"""Seeded synthetic inputs for the differentiable-LUT path (numpy only; no device code).

The generators never rely on a C++ standard-library distribution: wiring, tables and frames are drawn from
numpy's PCG64 stream so that the same seed gives the same arrays on every machine.  Layout is the FrameBuffer
one: node-major, frame-minor, ``[nodes, stride]`` with ``stride >= frames``; fp32 padding columns are zero and
padding bits of packed buffers are zero.
"""
import numpy as np

WAVE = 64


def frame_stride_fp32(frames, multiple=WAVE):
    """Row length (floats) of an fp32 frame buffer: frames rounded up to a wavefront multiple; rows whose byte length
    would be a multiple of 2 KiB get 128 more floats, because node rows that are a power of two apart fall into
    the same few L2 sets and the gathered rows then evict each other."""
    s = ((frames + multiple - 1) // multiple) * multiple
    if (s * 4) % 2048 == 0:
        s += 128
    return s


def frame_stride_bit(frames, multiple_bits=WAVE * 32):
    """Row length (32-bit words) of a bit-packed frame buffer: whole words for a wavefront, same de-aliasing pad."""
    s = ((frames + multiple_bits - 1) // multiple_bits) * (multiple_bits // 32)
    if (s * 4) % 2048 == 0:
        s += 96
    return s


def wiring(rng, input_nodes, output_nodes, n=6):
    """``[output_nodes, n]`` int32, each row n distinct input nodes drawn uniformly from [0, input_nodes)."""
    assert input_nodes >= n
    idx = rng.integers(0, input_nodes, size=(output_nodes, n), dtype=np.int64)
    while True:
        s = np.sort(idx, axis=1)
        bad = np.nonzero((s[:, 1:] == s[:, :-1]).any(axis=1))[0]
        if bad.size == 0:
            break
        idx[bad] = rng.integers(0, input_nodes, size=(bad.size, n), dtype=np.int64)
    return idx.astype(np.int32)


def uniform_frames(rng, nodes, frames, stride=None, lo=0.0, hi=1.0):
    stride = frame_stride_fp32(frames) if stride is None else stride
    a = np.zeros((nodes, stride), np.float32)
    a[:, :frames] = rng.random((nodes, frames), dtype=np.float32) * np.float32(hi - lo) + np.float32(lo)
    return a


def normal_frames(rng, nodes, frames, stride=None):
    stride = frame_stride_fp32(frames) if stride is None else stride
    a = np.zeros((nodes, stride), np.float32)
    a[:, :frames] = rng.standard_normal((nodes, frames), dtype=np.float32)
    return a


def pack_bits(bits, stride_words=None):
    """``[nodes, frames]`` of 0/1 -> ``[nodes, stride_words]`` int32, frame f at word f>>5, bit f&31."""
    nodes, frames = bits.shape
    words = (frames + 31) // 32
    stride_words = words if stride_words is None else stride_words
    padded = np.zeros((nodes, words * 32), np.uint8)
    padded[:, :frames] = bits
    packed = np.packbits(padded.reshape(nodes, words, 32), axis=2, bitorder="little")   # [nodes, words, 4] bytes
    out = np.zeros((nodes, stride_words), np.uint32)
    out[:, :words] = packed.view(np.uint32).reshape(nodes, words)
    return out.view(np.int32)


def unpack_bits(packed, frames):
    """inverse of :func:`pack_bits` -> ``[nodes, frames]`` uint8"""
    nodes = packed.shape[0]
    b = np.unpackbits(np.ascontiguousarray(packed).view(np.uint8).reshape(nodes, -1), axis=1, bitorder="little")
    return b[:, :frames]


def bernoulli_bits(rng, nodes, frames, stride_words=None, p=0.5):
    words = (frames + 31) // 32
    stride_words = words if stride_words is None else stride_words
    if p == 0.5:
        out = np.zeros((nodes, stride_words), np.uint32)
        out[:, :words] = rng.integers(0, 1 << 32, size=(nodes, words), dtype=np.uint32)
        tail = frames & 31
        if tail:
            out[:, words - 1] &= np.uint32((1 << tail) - 1)
        return out.view(np.int32)
    return pack_bits((rng.random((nodes, frames)) < p).astype(np.uint8), stride_words)


def truth_tables(rng, nodes):
    """``[nodes, 2]`` int32: 64-bit truth table per node, entries 0-31 in word 0."""
    return rng.integers(0, 1 << 32, size=(nodes, 2), dtype=np.uint32).view(np.int32)


def lut_tables(rng, nodes, n=6, lo=0.0, hi=1.0):
    return (rng.random((nodes, 1 << n), dtype=np.float32) * np.float32(hi - lo) + np.float32(lo)).astype(np.float32)
