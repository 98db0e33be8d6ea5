"""Module-swap helpers with the reference's names (segment_anything_fast/tools.py:1-36)."""


def replace_with_custom_fn_if_matches_filter(model, replacement_fn, filter_fn, cur_fqn="") -> None:
    """Walk `model`; every child for which filter_fn(child, fully_qualified_name)
    holds is replaced by replacement_fn(child), other children are searched
    recursively.  (tools.py:1-19)"""
    if cur_fqn == "":
        from .graphs import invalidate_recordings
        invalidate_recordings(model)  # recorded graphs hold the addresses of the modules replaced below
    for name, child in list(model.named_children()):
        fqn = name if cur_fqn == "" else f"{cur_fqn}.{name}"
        if filter_fn(child, fqn):
            setattr(model, name, replacement_fn(child))
        else:
            replace_with_custom_fn_if_matches_filter(child, replacement_fn, filter_fn, fqn)


def apply_eval_dtype_predictor(predictor, dtype=None):
    """eval() and optional dtype cast of the predictor's sub-models.  (tools.py:22-36)"""
    model = predictor.model
    for attr in ("image_encoder", "prompt_encoder", "mask_decoder"):
        sub = getattr(model, attr, None)
        if sub is None:
            continue
        sub = sub.eval()
        if dtype is not None:
            sub = sub.to(dtype)
        setattr(model, attr, sub)
    return predictor
