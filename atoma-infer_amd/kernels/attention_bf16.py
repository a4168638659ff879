"""bfloat16 attention over the paged cache on the matrix cores."""
from __future__ import annotations


def try_attention(q, k_cache, v_cache, out, ctx, cache, scale, window, nh, nkv, hd) -> bool:
    """Run the fast kernels if they take this shape; False sends the caller to the general kernel."""
    return False
