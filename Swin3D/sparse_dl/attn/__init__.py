from . import attn_coff  # noqa: F401
