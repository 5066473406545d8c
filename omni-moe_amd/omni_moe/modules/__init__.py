from .omni_moe import OmniMoE, OmniMoEConfig  # noqa: F401
