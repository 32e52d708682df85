"""Which call sites take their FP8 activation straight from the norm kernel instead of launching the 1-D
quantiser on the norm's bf16 output (batchgen/models/glm/glm5/norm_quant_fuse_policy.py:57-105).  The fused kernel
gives the same bytes and scales as the two launches, so the switch changes launches, never values.  Pure Python on
purpose: graph-segment code reads it at import time on machines without a GPU.

Of the three sites only ``shared_expert`` lies on the path this package serves (add + RMSNorm -> the dense
expert's / the MoE layer's ``x_fp8`` / ``x_scale``); ``qkv_a`` and ``q_a`` belong to attention and are listed so
that callers written against the reference's names keep working.
"""

GLM5_NORM_QUANT_FUSE_SITES = ("qkv_a", "q_a", "shared_expert")

# Master switch; False = every site quantises with its own launch.
GLM5_NORM_QUANT_FUSE = True

# Sites that keep their own quantiser launch while the master switch is on.
GLM5_NORM_QUANT_FUSE_DISABLED_SITES: tuple = ()


def glm5_norm_quant_fuse_enabled() -> bool:
    if type(GLM5_NORM_QUANT_FUSE) is not bool:
        raise TypeError(f"GLM5_NORM_QUANT_FUSE must be True or False, got {GLM5_NORM_QUANT_FUSE!r} "
                        f"({type(GLM5_NORM_QUANT_FUSE).__name__})")
    return GLM5_NORM_QUANT_FUSE


def glm5_norm_quant_fuse_site_enabled(site: str) -> bool:
    """Unknown names raise (here and in the opt-out list): a misspelt site must not silently keep its launch."""
    known = GLM5_NORM_QUANT_FUSE_SITES
    if site not in known:
        raise ValueError(f"unknown norm/quant fusion site {site!r}; known sites are {known}")
    off = GLM5_NORM_QUANT_FUSE_DISABLED_SITES
    if not isinstance(off, (tuple, list, frozenset, set)):
        raise TypeError(f"GLM5_NORM_QUANT_FUSE_DISABLED_SITES must be a tuple of site names, got {off!r} "
                        f"({type(off).__name__})")
    strangers = [s for s in off if s not in known]
    if strangers:
        raise ValueError(f"GLM5_NORM_QUANT_FUSE_DISABLED_SITES names unknown sites {strangers}; known sites are "
                         f"{known}")
    return glm5_norm_quant_fuse_enabled() and site not in off
