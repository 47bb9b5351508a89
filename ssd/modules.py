"""Drop-in for the reference module of the same path."""
from bi_mamba2_amd.modules import BiMamba2  # noqa: F401
