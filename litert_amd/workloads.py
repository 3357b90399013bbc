"""Seeded synthetic inputs for the five benchmark / parity configurations.

Shapes, distributions and quantization parameters are the ones the benchmark
contract names; every tensor draws from its own numpy Generator stream so that a
configuration is reproducible from (seed, name) alone. Arrays are numpy, host side.
"""
import numpy as np

SEED = 0x5EED


def _rng(name, seed=SEED):
    return np.random.default_rng([seed, *[ord(c) for c in name]])


def pack_int4(w):
    """[N, K] int8 in [-8, 7] -> [N, K/2] uint8, low nibble = even k."""
    w = np.asarray(w, np.int8)
    lo = w[:, 0::2].astype(np.uint8) & 0xF
    hi = w[:, 1::2].astype(np.uint8) & 0xF
    return (lo | (hi << 4)).astype(np.uint8)


def int8_fc(batches=1, depth=2048, out_depth=2048, in_scale=0.02, in_zp=-3, out_scale=0.05,
            out_zp=5, seed=SEED):
    """Config 1 (and, with other sizes, config 4): full-integer per-channel int8 FC."""
    x = _rng("x", seed).integers(-128, 128, (batches, depth)).astype(np.int8)
    w = _rng("w", seed).integers(-127, 128, (out_depth, depth)).astype(np.int8)
    w_scale = np.exp(_rng("ws", seed).uniform(np.log(1e-3), np.log(1e-2), out_depth)).astype(
        np.float32)
    bias = _rng("bias", seed).integers(-2 ** 14, 2 ** 14 + 1, out_depth).astype(np.int32)
    return dict(x=x, w=w, w_scale=w_scale, bias=bias, in_scale=np.float32(in_scale), in_zp=in_zp,
                out_scale=np.float32(out_scale), out_zp=out_zp)


def prefill_int8_fc(batches=2048, depth=4096, out_depth=4096, seed=SEED):
    """Config 4: prefill-shaped int8 GEMM, input scale 0.03 / zero point 0."""
    return int8_fc(batches, depth, out_depth, in_scale=0.03, in_zp=0, out_scale=0.05, out_zp=0,
                   seed=seed)


def hybrid_fc(batches=1, depth=4096, out_depth=14336, seed=SEED):
    """Config 2: float activations N(0,1), int8 per-channel weights, no bias."""
    x = _rng("x", seed).standard_normal((batches, depth)).astype(np.float32)
    w = _rng("w", seed).integers(-127, 128, (out_depth, depth)).astype(np.int8)
    pcs = _rng("pcs", seed).uniform(2e-3, 8e-3, out_depth).astype(np.float32)
    return dict(x=x, w=w, pcs=pcs)


def blockwise_int4_fc(batches=1, depth=4096, out_depth=14336, blocksize=32, seed=SEED,
                      lo=-7, hi=7):
    """Config 3 (and each node of config 5): int4 weights in [-7, 7], fp16 block scales."""
    x = _rng("x", seed).standard_normal((batches, depth)).astype(np.float32)
    w = _rng("w", seed).integers(lo, hi + 1, (out_depth, depth)).astype(np.int8)
    scales = _rng("s", seed).uniform(5e-3, 2e-2, (out_depth, depth // blocksize)).astype(
        np.float16)
    return dict(x=x, w=w, packed=pack_int4(w), scales=scales, blocksize=blocksize)


# Config 5: the seven FULLY_CONNECTED nodes of one Gemma-2B-shaped decoder layer (in, out).
GEMMA2B_LAYER_FCS = [("q_proj", 2048, 2048), ("k_proj", 2048, 256), ("v_proj", 2048, 256),
                     ("o_proj", 2048, 2048), ("gate_proj", 2048, 16384),
                     ("up_proj", 2048, 16384), ("down_proj", 16384, 2048)]
GEMMA2B_LAYERS = 18
