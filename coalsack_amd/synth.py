"""Synthetic MoE-layer inputs with the distributions the benchmark configs name.

MXFP4 bytes come from the same counter-based generator the library runs on the
GPU (csk_layer_fill_synthetic), so a host can replay any (layer, expert,
matrix) slice without ever holding a whole layer; float tensors are drawn on
the host with numpy and uploaded.
"""
import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def mix64(z):
    """splitmix64 finaliser on uint64 arrays (wraps modulo 2^64)."""
    z = np.asarray(z, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = z + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def stream_key(seed, layer, expert, which):
    with np.errstate(over="ignore"):
        inner = mix64(np.uint64(layer) * np.uint64(1000003) + np.uint64(expert) * np.uint64(16)
                      + np.uint64(which))
        return mix64(np.uint64(seed) ^ inner)


def mxfp4_blocks(seed, layer, expert, which, rows, K, scale_lo=117, scale_span=5):
    """The [rows, K] matrix of stream (seed, layer, expert, which) as 17-byte blocks
    in the reference's storage format (scale byte, then 16 quant bytes)."""
    nb = rows * (K // 32)
    key = stream_key(seed, layer, expert, which)
    b = np.arange(nb, dtype=np.uint64)
    with np.errstate(over="ignore"):
        h0 = mix64(key + np.uint64(3) * b)
        h1 = mix64(key + np.uint64(3) * b + np.uint64(1))
        h2 = mix64(key + np.uint64(3) * b + np.uint64(2))
    out = np.empty((nb, 17), np.uint8)
    out[:, 0] = (scale_lo + (h0 >> np.uint64(33)) % np.uint64(scale_span)).astype(np.uint8)
    out[:, 1:9] = h1.astype("<u8").view(np.uint8).reshape(nb, 8)
    out[:, 9:17] = h2.astype("<u8").view(np.uint8).reshape(nb, 8)
    return out.reshape(-1)


class LayerInputs:
    """Float tensors of one layer (router, biases, norm) + geometry."""

    def __init__(self, E, k, H, F, seed=1234, layer=0, hot_experts=0, hot_offset=2.0,
                 with_norm=False):
        self.E, self.k, self.H, self.F, self.seed, self.layer = E, k, H, F, seed, layer
        rng = np.random.default_rng([seed, layer, 7])
        self.gate_w = rng.normal(0.0, 0.02, (E, H)).astype(np.float32)
        self.gate_b = rng.normal(0.0, 0.01, E).astype(np.float32)
        if hot_experts:
            hot = rng.choice(E, hot_experts, replace=False)
            self.gate_b[hot] += np.float32(hot_offset)
        self.b_up = rng.normal(0.0, 0.01, (E, F)).astype(np.float32)
        self.b_gate = rng.normal(0.0, 0.01, (E, F)).astype(np.float32)
        self.b_down = rng.normal(0.0, 0.01, (E, H)).astype(np.float32)
        self.norm_w = rng.normal(1.0, 0.02, H).astype(np.float32) if with_norm else None

    def blocks(self, e, which):
        rows, K = (self.H, self.F) if which == 2 else (self.F, self.H)
        return mxfp4_blocks(self.seed, self.layer, e, which, rows, K)


def hidden_states(T, H, seed=99):
    return np.random.default_rng([seed, T]).normal(0.0, 1.0, (T, H)).astype(np.float32)
