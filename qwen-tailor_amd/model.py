"""Model shape constants the hot path is specialised for (qwen35/model.py:35-60)."""
from dataclasses import dataclass


@dataclass
class Cfg:
    hidden: int = 1024
    inter: int = 3584
    vocab: int = 248320
    layers: int = 24
    eps: float = 1e-6
    # full attention
    n_heads: int = 8
    n_kv: int = 2
    head_dim: int = 256
    rope_dim: int = 64
    rope_theta: float = 1e7
    # linear attention
    hk: int = 16
    hv: int = 16
    dk: int = 128
    dv: int = 128
    conv_k: int = 4

    @property
    def conv_dim(self):
        return 2 * self.hk * self.dk + self.hv * self.dv

    def is_linear(self, i):
        return (i + 1) % 4 != 0
