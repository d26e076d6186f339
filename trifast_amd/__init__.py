"""trifast_amd: fused triangle self-attention for AMD Instinct MI355X (gfx950).

Same Python surface as the reference package (src/trifast/__init__.py:1-3), plus an
ending-node entry on untransposed tensors and, in ``trifast_amd.nn``, the gated block
that calls the operator in AlphaFold-style models.
"""

from trifast_amd.torch import triangle_attention, triangle_attention_ending_node

__version__ = "0.1.13"

__all__ = ["triangle_attention", "triangle_attention_ending_node"]
