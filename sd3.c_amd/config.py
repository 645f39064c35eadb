"""Hyper-parameters of the denoiser, mirrored 1:1 from the positional scalars of the reference's
`DiT_forward` (modules.cpp:1611-1613) and `DiT_block_forward` (modules.cpp:1514)."""
from dataclasses import dataclass, field
from typing import Tuple


@dataclass(frozen=True)
class DiTConfig:
    num_layers: int = 24
    dual_attention_layers: Tuple[int, ...] = tuple(range(13))
    pooled_dim: int = 2048
    captions_dim: int = 4096
    in_channels: int = 16
    emb_dim: int = 1536
    attn_heads: int = 24
    mlp_expand: int = 4
    patch_size: int = 2
    pos_embed_max_size: int = 384
    base_height: int = 128
    use_qk_norm: bool = True

    @property
    def head_dim(self) -> int:
        return self.emb_dim // self.attn_heads

    def tokens(self, H: int, W: int) -> int:
        p = self.patch_size
        return ((H - p) // p + 1) * ((W - p) // p + 1)


def sd35_medium() -> DiTConfig:
    """SD3.5-medium MMDiT-X shape: 24 blocks at width 1536, the first 13 with the extra image self-attention."""
    return DiTConfig()


def reference_dit_test() -> DiTConfig:
    """The configuration of the reference's own full-model check (module_tests/DiT.py:8-21)."""
    return DiTConfig(num_layers=3, dual_attention_layers=(0,), pooled_dim=2048, captions_dim=2048, in_channels=16, emb_dim=256,
                     attn_heads=2, mlp_expand=4, patch_size=2, pos_embed_max_size=96, base_height=64, use_qk_norm=True)
