"""Seeded synthetic inputs for the MoE layer, at the shapes of the benchmark
configurations.  Shared by the tests, the benchmark and the fixture script so
that every consumer sees identical values for a given (config, seed).

Value distributions follow the benchmark configurations: activations N(0,1)
(RMS-normalised per row for the bf16 configs), weights N(0,0.02), expert
biases N(0,0.02), router bias N(0,0.1).  For bf16 configs every tensor is
rounded to the nearest bf16 (ties to even) and returned as float32 holding
exactly representable values, which is the host layout the upload entry point
takes (reference: run.cpp:234-247 keeps fp32 on the host).
"""
from __future__ import annotations

import concurrent.futures
import dataclasses
import hashlib
import os

import numpy as np


@dataclasses.dataclass(frozen=True)
class LayerShape:
    name: str
    tokens: int
    hidden: int
    inter: int
    experts: int
    topk: int = 4
    limit: float = 7.0
    bf16: bool = True
    zipf: float = 0.0  # >0: router bias follows Zipf(s) popularity


CONFIGS = {
    # the reference's CPU-runnable case (fp32)
    "c1": LayerShape("c1", 64, 256, 256, 8, bf16=False),
    # GPT-OSS-20B shape, the configuration the headline metric is quoted on
    "c2": LayerShape("c2", 4096, 2880, 2880, 32),
    # skewed routing at the 20B shape
    "c3a": LayerShape("c3a", 512, 2880, 2880, 32, zipf=1.2),
    "c3b": LayerShape("c3b", 7168, 2880, 2880, 32, zipf=1.2),
    # GPT-OSS-120B shape
    "c4": LayerShape("c4", 6144, 2880, 2880, 128),
    # 20B shape, expert matrices given as MXFP4 blocks and scales (make_experts_mxfp4)
    "c5": LayerShape("c5", 64, 2880, 2880, 32),
    # Not a benchmark configuration: a yardstick.  Four experts and top-4, so every
    # token goes to every expert and the grouped GEMMs are four dense ones of
    # 4096 rows each: what the kernels reach without ragged segments.
    "d4": LayerShape("d4", 4096, 2880, 2880, 4),
}


def round_bf16(a: np.ndarray) -> np.ndarray:
    """float32 -> nearest bf16 (ties to even), returned as float32."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32)
    finite = (~u & np.uint32(0x7F800000)) != 0
    r = u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    u = np.where(finite, r, u) & np.uint32(0xFFFF0000)
    return u.view(np.float32)


def to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """float32 holding bf16-representable values -> uint16 bit patterns."""
    return (round_bf16(a).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def _round_bf16_inplace(chunk: np.ndarray) -> None:
    """In-place variant of round_bf16 for finite values."""
    u = chunk.view(np.uint32)
    lsb = u >> np.uint32(16)
    lsb &= np.uint32(1)
    lsb += np.uint32(0x7FFF)
    u += lsb
    u &= np.uint32(0xFFFF0000)


_CHUNK = 1 << 22


def _normal(seed, stream, shape, std, bf16):
    """N(0, std) values of the given shape.  Every chunk of _CHUNK elements has
    a PCG64 stream of its own keyed by (seed, stream, chunk index), so the
    result does not depend on how many worker threads fill the chunks."""
    n = int(np.prod(shape))
    out = np.empty(n, dtype=np.float32)

    def fill(ci):
        chunk = out[ci * _CHUNK:(ci + 1) * _CHUNK]
        g = np.random.Generator(np.random.PCG64(np.random.SeedSequence([seed, stream, ci])))
        g.standard_normal(chunk.shape[0], dtype=np.float32, out=chunk)
        chunk *= np.float32(std)
        if bf16:
            _round_bf16_inplace(chunk)

    nchunks = (n + _CHUNK - 1) // _CHUNK
    if nchunks <= 2:
        for ci in range(nchunks):
            fill(ci)
    else:
        workers = min(16, os.cpu_count() or 1)
        with concurrent.futures.ThreadPoolExecutor(workers) as pool:
            list(pool.map(fill, range(nchunks)))
    return out.reshape(shape)


def zipf_popularity(experts: int, s: float) -> np.ndarray:
    p = np.arange(1, experts + 1, dtype=np.float64) ** (-s)
    return p / p.sum()


def make_activations(shape: LayerShape, seed: int = 0, tokens: int | None = None) -> np.ndarray:
    T = shape.tokens if tokens is None else tokens
    x = _normal(seed, 1, (T, shape.hidden), 1.0, False)
    if shape.bf16:
        ms = np.mean(x.astype(np.float64) ** 2, axis=1, keepdims=True)
        x = round_bf16((x / np.sqrt(ms + 1e-5)).astype(np.float32))
    return x


def make_router(shape: LayerShape, seed: int = 0):
    wr = _normal(seed, 2, (shape.experts, shape.hidden), 0.02, shape.bf16)
    br = _normal(seed, 3, (shape.experts,), 0.1, False)
    if shape.zipf > 0:
        # A token takes an expert at most once, so the head of Zipf(s) cannot be
        # met (p_1 * K > 1): the target is the water-filled one, min(1, .) per
        # token with the excess spread over the tail in proportion.  Logits
        # spread by about sigma = 0.02*sqrt(H); bias = c*sigma*log(p) with
        # c = 0.65 minimises both the L1 and the KL distance of the realised
        # top-4 histogram to that target (scanned in steps of 0.05 at T = 7168).
        c = 0.65 * 0.02 * np.sqrt(shape.hidden)
        br = (br + c * np.log(zipf_popularity(shape.experts, shape.zipf))).astype(np.float32)
    if shape.bf16:
        br = round_bf16(br)
    return wr, br.astype(np.float32)


def make_experts(shape: LayerShape, seed: int = 0):
    E, H, IM = shape.experts, shape.hidden, shape.inter
    w1 = _normal(seed, 4, (E, 2 * IM, H), 0.02, shape.bf16)
    b1 = _normal(seed, 5, (E, 2 * IM), 0.02, shape.bf16)
    w2 = _normal(seed, 6, (E, H, IM), 0.02, shape.bf16)
    b2 = _normal(seed, 7, (E, H), 0.02, shape.bf16)
    return w1, b1, w2, b2


def make_experts_mxfp4(shape: LayerShape, seed: int = 0):
    """MXFP4 expert matrices: per 32 weights 16 random bytes (uniform nibbles) and
    a scale byte uniform in [119, 129] (exponents -8 .. 2); biases as make_experts.
    Returns (w1_blocks, w1_scales, b1, w2_blocks, w2_scales, b2) with blocks
    u8 [E, rows, cols/32, 16] and scales u8 [E, rows, cols/32]."""
    E, H, IM = shape.experts, shape.hidden, shape.inter
    rng = np.random.Generator(np.random.PCG64([seed, 40]))
    w1_blocks = rng.integers(0, 256, (E, 2 * IM, H // 32, 16), dtype=np.uint8)
    w1_scales = rng.integers(119, 130, (E, 2 * IM, H // 32), dtype=np.uint8)
    w2_blocks = rng.integers(0, 256, (E, H, IM // 32, 16), dtype=np.uint8)
    w2_scales = rng.integers(119, 130, (E, H, IM // 32), dtype=np.uint8)
    b1 = _normal(seed, 5, (E, 2 * IM), 0.02, shape.bf16)
    b2 = _normal(seed, 7, (E, H), 0.02, shape.bf16)
    return w1_blocks, w1_scales, b1, w2_blocks, w2_scales, b2


def make_layer(shape: LayerShape, seed: int = 0, tokens: int | None = None) -> dict:
    x = make_activations(shape, seed, tokens)
    wr, br = make_router(shape, seed)
    w1, b1, w2, b2 = make_experts(shape, seed)
    pos = np.zeros(x.shape[0], dtype=np.int32)
    return dict(x=x, pos=pos, w_router=wr, b_router=br, w_mlp1=w1, b_mlp1=b1,
                w_mlp2=w2, b_mlp2=b2)


def digest(*arrays: np.ndarray) -> str:
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()
