"""Drop-in for the reference module of the same path (gated RMS norm and LayerNorm: rmsnorm_fn, layernorm_fn, RMSNorm, LayerNorm, LayerNormFn): names come from bi_mamba2_amd.layernorm_gated."""
from bi_mamba2_amd.layernorm_gated import LayerNorm, LayerNormFn, RMSNorm, layernorm_fn, rmsnorm_fn  # noqa: F401
