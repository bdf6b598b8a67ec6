"""Seeded synthetic inputs of the five benchmark configurations.

All arrays are produced with numpy's PCG64 generator from the stated seeds, so
every host with the same numpy builds identical bits.  The weight-side
quantizer is harness code (the library receives already-quantized codes):
symmetric per output channel, scale = absmax / qmax (1 for an all-zero
channel), code = clamp(round_half_away(w / scale), -qmax, qmax).
"""
import numpy as np


def _round_half_away(x):
    return np.sign(x) * np.floor(np.abs(x) + 0.5)


def quantize_weight(w_out_in, qmax):
    """w_out_in: fp32 [N_out, K_in].  Returns (B[K, N] int8 codes, scale[N] fp32)."""
    w = np.asarray(w_out_in, np.float32)
    absmax = np.abs(w).max(axis=1)
    scale = np.where(absmax > 0, absmax / np.float32(qmax), np.float32(1.0)).astype(np.float32)
    codes = _round_half_away(w.astype(np.float64) / scale[:, None].astype(np.float64))
    codes = np.clip(codes, -qmax, qmax).astype(np.int8)
    return np.ascontiguousarray(codes.T), scale


def normal_f32(seed, shape, std=1.0):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def normal_f16_bits(seed, shape):
    """fp16 N(0,1) as raw binary16 bit patterns (uint16)."""
    return normal_f32(seed, shape).astype(np.float16).view(np.uint16)


def w8a8_case(M, K, N, seed_w, seed_a):
    """Configs 0 and 1: fp32 N(0, 0.02) weights [N, K] -> per-channel int8; fp16 N(0,1) A."""
    B, s = quantize_weight(normal_f32(seed_w, (N, K), 0.02), 127)
    return dict(M=M, K=K, N=N, B=B, w_scale=s, A=normal_f16_bits(seed_a, (M, K)))


def w4a8_case(M, K, N, seed_w, seed_a, outlier_fraction=0.005, outlier_gain=20.0):
    """Config 2: int4 [-7,7] weights; fp16 A with a fraction of entries x20."""
    B, s = quantize_weight(normal_f32(seed_w, (N, K), 0.02), 7)
    rng = np.random.default_rng(seed_a)
    a = rng.standard_normal((M, K), dtype=np.float32)
    mask = rng.random((M, K), dtype=np.float32) < np.float32(outlier_fraction)
    a = np.where(mask, a * np.float32(outlier_gain), a).astype(np.float16)
    return dict(M=M, K=K, N=N, B=B, w_scale=s, A=a.view(np.uint16))


def ffn_case(M, H, I, seeds=(6, 7, 8, 9)):
    """Config 3: gate, up [I, H] and down [H, I] int4 per-channel; x fp32 [M, H]
    (fp16-rounded values, since the FFN entry point takes fp32)."""
    Bg, sg = quantize_weight(normal_f32(seeds[0], (I, H), 0.02), 7)
    Bu, su = quantize_weight(normal_f32(seeds[1], (I, H), 0.02), 7)
    Bd, sd = quantize_weight(normal_f32(seeds[2], (H, I), 0.02), 7)
    x = normal_f32(seeds[3], (M, H)).astype(np.float16).astype(np.float32)
    return dict(M=M, H=H, I=I, B_gu=np.ascontiguousarray(np.concatenate([Bg, Bu], axis=1)),
                s_gu=np.concatenate([sg, su]), B_down=Bd, s_down=sd, x=x)


def moe_case(T, H, E, top_k, I, seeds=(10, 11, 12, 13, 14)):
    """Config 4: router logits N(0,1) -> softmax -> top-k (ties to the lower index)
    -> renormalised coefficients; expert gate/up [H, 2I] and down [I, H] int8."""
    logits = normal_f32(seeds[0], (T, E)).astype(np.float64)
    p = np.exp(logits - logits.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    order = np.argsort(-p, axis=1, kind="stable")[:, :top_k]
    w = np.take_along_axis(p, order, axis=1)
    w = (w / w.sum(axis=1, keepdims=True)).astype(np.float32)
    experts = []
    rg = np.random.default_rng(seeds[1])
    ru = np.random.default_rng(seeds[2])
    rd = np.random.default_rng(seeds[3])
    for _ in range(E):
        Bg, sg = quantize_weight(rg.standard_normal((I, H), dtype=np.float32) * np.float32(0.02), 127)
        Bu, su = quantize_weight(ru.standard_normal((I, H), dtype=np.float32) * np.float32(0.02), 127)
        Bd, sd = quantize_weight(rd.standard_normal((H, I), dtype=np.float32) * np.float32(0.02), 127)
        experts.append((np.ascontiguousarray(np.concatenate([Bg, Bu], axis=1)),
                        np.concatenate([sg, su]), Bd, sd))
    x = normal_f32(seeds[4], (T, H)).astype(np.float16).astype(np.float32)
    return dict(T=T, H=H, E=E, top_k=top_k, I=I, ids=order.astype(np.int32), routes=w,
                experts=experts, x=x)


# The five configurations at full size.
CONFIGS = {
    0: lambda: w8a8_case(64, 2048, 2048, 0, 1),
    1: lambda: w8a8_case(1, 4096, 14336, 2, 3),
    2: lambda: w4a8_case(2048, 4096, 4096, 4, 5),
    3: lambda: ffn_case(128, 4096, 14336),
    4: lambda: moe_case(256, 2048, 32, 4, 1024),
}
