"""Independent float64 statements of the per-layer math, written the textbook way (numpy vectorised,
complex rotations, fancy-index scatters).  They share no code and no loop structure with the C oracle
and exist to pin it; they are also what tests/golden/make_golden.py evaluates."""
import numpy as np


def rmsnorm64(x, gamma, eps):
    x = np.asarray(x, np.float64)
    ms = np.mean(x * x, axis=-1, keepdims=True)
    return x / np.sqrt(ms + eps) * np.asarray(gamma, np.float64)


def fused_norm64(residual, out, bias, gamma, eps, residual_excludes_bias=False):
    x = np.asarray(out, np.float64)
    if residual is not None:
        x = x + np.asarray(residual, np.float64)
    stored = x.copy()
    if bias is not None:
        x = x + np.asarray(bias, np.float64)
    if not residual_excludes_bias:
        stored = x.copy()
    return (stored if residual is not None else None), rmsnorm64(x, gamma, eps)


def swiglu64(x):
    x = np.asarray(x, np.float64)
    gate, up = x[:, 0, :], x[:, 1, :]
    return gate * (1.0 / (1.0 + np.exp(-gate))) * up


def rope_angles64(timesteps, head_size, rotary_dim, base):
    """angles [len(timesteps), head_size/2]; zero where the pair is not rotated."""
    half = head_size // 2
    d = np.arange(half, dtype=np.float64)
    inv = np.where(d < rotary_dim // 2, base ** (-(2.0 * d) / rotary_dim), 0.0)
    return np.asarray(timesteps, np.float64)[:, None] * inv[None, :]


def rotate_half64(x, angles):
    """x [..., head_size] rotated pairwise (d, d + head_size/2) by angles [..., head_size/2], as a
    complex multiplication (x_d + i x_{d+half}) * exp(i angle)."""
    x = np.asarray(x, np.float64)
    half = x.shape[-1] // 2
    z = (x[..., :half] + 1j * x[..., half:]) * np.exp(1j * angles)
    return np.concatenate([z.real, z.imag], axis=-1)


def qkv_rope64(qkv, bias, padding_offset, history_length, batch, seq_len, head_num, kv_head_num,
               rotary_dim, base, fill=0.0):
    """Returns q, k, v (float64, padded positions = fill) and the boolean mask of written (b, s)."""
    qkv = np.asarray(qkv, np.float64)
    tokens, qkv_heads, hs = qkv.shape
    if bias is not None:
        qkv = qkv + np.asarray(bias, np.float64).reshape(1, qkv_heads, hs)
    p = np.arange(tokens) + np.asarray(padding_offset[:tokens], np.int64)
    b, s = p // seq_len, p % seq_len
    t = np.asarray(history_length, np.int64)[b] + s
    ang = rope_angles64(t, hs, rotary_dim, base)[:, None, :]          # [tokens, 1, half]
    qh = rotate_half64(qkv[:, :head_num], ang)
    kh = rotate_half64(qkv[:, head_num:head_num + kv_head_num], ang)
    vh = qkv[:, head_num + kv_head_num:]
    q = np.full((batch, head_num, seq_len, hs), fill, np.float64)
    k = np.full((batch, kv_head_num, seq_len, hs), fill, np.float64)
    v = np.full((batch, kv_head_num, seq_len, hs), fill, np.float64)
    q[b, :, s, :] = qh
    k[b, :, s, :] = kh
    v[b, :, s, :] = vh
    written = np.zeros((batch, seq_len), bool)
    written[b, s] = True
    return q, k, v, written
