"""Model families: Llama-3 (8B/70B), Mixtral 8x7B (MoE), GPT-2 — one shard-aware decoder — and
Nesizen, a heterogeneous stack of attention / gated-linear-attention layers (models/nesizen.py),
Zinesun, latent-attention layers on a post-norm residual (models/zinesun.py), and Lizizen, parallel
layers with a token shift over distance-biased and differential attention (models/lizizen.py), and
Gevipel, sandwich-normed layers over sloped window attention, the gated delta rule and latent
attention with a sink, with routed plain experts (models/gevipel.py)."""
from .shard import LocalDims, Shard, local_dims  # noqa: F401
from .transformer import LogicalParam, TransformerLM  # noqa: F401
from .nesizen import NesizenLM  # noqa: F401
from .zinesun import ZinesunLM  # noqa: F401
from .lizizen import LizizenLM  # noqa: F401
from .gevipel import GevipelLM  # noqa: F401


class LlamaForCausalLM(TransformerLM):
    """Llama-3 family (GQA, RoPE theta 5e5, RMSNorm, SwiGLU)."""


class MixtralForCausalLM(TransformerLM):
    """Mixtral (Llama attention + top-2 of 8 SwiGLU experts, dense-dispatch MoE)."""


class GPT2LMHeadModel(TransformerLM):
    """GPT-2 (learned positions, LayerNorm, GELU MLP with biases, tied embeddings)."""


_ARCH = {"llama": LlamaForCausalLM, "mixtral": MixtralForCausalLM, "gpt2": GPT2LMHeadModel,
         "nesizen": NesizenLM, "zinesun": ZinesunLM, "lizizen": LizizenLM, "gevipel": GevipelLM}


def supports_f32(arch: str) -> bool:
    """Whether the family's GPU kernels have a true 32-bit form (EngineConfig.dtype = "fp32")."""
    return bool(getattr(_ARCH[arch], "supports_f32", False))


def build_model(cfg, shard=None, device="cpu", dtype=None, comm=None):
    import torch

    cls = _ARCH[cfg.arch]
    return cls(cfg, shard or Shard(), device=device, dtype=dtype or torch.bfloat16, comm=comm)
