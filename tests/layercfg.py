"""Decoder-layer configurations shared by the layer tests, smoke and bench (argument packing of
zkp_layer_create / orc_layer)."""
import numpy as np


def pack(seq, embed, heads, hidden, sf_linear, sf_gate, sf_attn, bs, L, M, sf_in, thetas, swiglu_low, swiglu_len, swiglu_in_scale,
         swiglu_out_scale=16.0, rms_eps=1e-5, value_scale=65536.0, open_weights=True, head_group=0):
    cu = np.array([seq, embed, heads, hidden, sf_linear, sf_gate, sf_attn, L, M, swiglu_len, 1 if open_weights else 0, len(bs)] + list(bs) + [head_group], dtype=np.uint32)
    cf = np.array([float(sf_in), float(swiglu_low), float(swiglu_in_scale), float(swiglu_out_scale), rms_eps, float(value_scale)] + [float(t) for t in thetas], dtype=np.float64)
    return cu, cf


def llama7b(seq=2048, open_weights=True, head_group=0):
    """the reference drivers' constants (self-attn.cu:47-49,87-88, ffn.cu:47-54) at the LLaMa-2-7B shape; head_group = g proves
    attention g heads at a time with zkAttnStacked, 0 head by head"""
    return pack(seq, 4096, 32, 11008, 1 << 16, 1 << 20, 1 << 20, [1 << 8, 1 << 20, 1 << 20], 1, 0, 1 << 32, [1 << 18, 1 << 22],
                -(1 << 21), 1 << 22, 4096.0, open_weights=open_weights, head_group=head_group)


def tiny(open_weights=True, head_group=0):
    """16 tokens, width 32, 2 heads, hidden 64; fixed-point scale 2^8 throughout so every lookup table fits its tensor"""
    return pack(16, 32, 2, 64, 1 << 8, 1 << 10, 1 << 7, [1 << 8, 1 << 8, 1 << 8], 1, 0, 1 << 16, [1 << 6, 1 << 8],
                -512, 1024, 64.0, value_scale=256.0, open_weights=open_weights, head_group=head_group)


def tiny_weights(seed, cu, w_std=0.25, w_scale=256):
    rng = np.random.default_rng(seed)
    E, Hd = int(cu[1]), int(cu[3])
    mk = lambda i, o: np.round(rng.normal(0, w_std, (i, o)) * w_scale).astype(np.int32)
    norm = lambda: np.full((1, E), w_scale, dtype=np.int32)
    return [norm(), mk(E, E), mk(E, E), mk(E, E), mk(E, E), norm(), mk(E, Hd), mk(E, Hd), mk(Hd, E)]
