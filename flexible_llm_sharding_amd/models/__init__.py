

def hybrid_family(cfg):
    """The module of a stateful hybrid family (``cfg.family``): ``layout`` / ``placements`` of a layer's
    weight image, ``run_layer`` on a step batch, ``layer_flops``, and ``state_spec``, what a request
    keeps between steps."""
    fam = getattr(cfg, "family", "dense")
    if fam == "kagolix":
        from . import kagolix
        return kagolix
    if fam == "sisavik":
        from . import sisavik
        return sisavik
    if fam == "gizezen":
        from . import gizezen
        return gizezen
    if fam == "lopilix":
        from . import lopilix
        return lopilix
    raise NotImplementedError(f"no hybrid family {fam!r}")
