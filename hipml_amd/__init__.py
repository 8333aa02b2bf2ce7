"""hipml_amd: MI355X (gfx950) implementation of hipml's full-attention hot path.

`hipml_amd.attn` mirrors the reference's launcher interface over the C ABI of
libhipml_attn.so (include/hipml_attn.h); `hipml_amd.build` compiles it.
"""
from . import attn  # noqa: F401
from .attn import HipmlError, DeepKv  # noqa: F401
