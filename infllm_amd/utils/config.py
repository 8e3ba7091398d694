"""Run configuration in the reference's YAML layout (config/*.yaml; benchmark/pred.py:22-40).

The reference reads the file with OmegaConf, merges ``key.sub=value`` command-line overrides into it, and fills
two defaults: ``model.tokenizer_path`` (the model path) and ``truncation`` (none).  Its ``model`` section is then
handed to ``patch_hf`` wholesale - ``patch_hf(model, conf.model.type, **conf.model)`` (pred.py:54-56) - so the
section's keys are the attention type's knobs (``block_size``, ``n_init``, ``n_local``, ``topk``, ``repr_topk``,
``max_cached_block``, ``exc_block_size``, ``fattn``, ``base``, ``distance_scale``, ...) next to ``type`` and
``path``.  OmegaConf is not a dependency here: PyYAML's safe loader and a dict with attribute access do the same.
"""
import yaml


class Section(dict):
    """dict whose keys also read as attributes (``conf.model.topk``); ``**section`` spreads the keys."""

    def __getattr__(self, name):
        try:
            return self[name]
        except KeyError:
            raise AttributeError(name) from None

    def __setattr__(self, name, value):
        self[name] = value


def _wrap(node):
    if isinstance(node, dict):
        return Section((k, _wrap(v)) for k, v in node.items())
    if isinstance(node, list):
        return [_wrap(v) for v in node]
    return node


def load_config(path, overrides=()):
    """YAML file -> nested ``Section``; ``overrides`` are ``"model.topk=32"`` strings (values parsed as YAML scalars,
    missing sections created), applied after the file as the reference's command line is."""
    with open(path) as f:
        conf = _wrap(yaml.safe_load(f) or {})
    if not isinstance(conf, Section):
        raise ValueError(f"{path}: the top level of a configuration must be a mapping")
    for item in overrides:
        key, sep, text = item.partition("=")
        if not sep or not key:
            raise ValueError(f"override {item!r} is not of the form key.sub=value")
        node = conf
        *parents, leaf = key.lstrip("-").split(".")
        for name in parents:
            if not isinstance(node.get(name), Section):
                node[name] = Section()
            node = node[name]
        node[leaf] = _wrap(yaml.safe_load(text)) if text != "" else None
    model = conf.get("model")
    if not isinstance(model, Section) or "type" not in model:
        raise ValueError(f"{path}: no model section with a type")
    if "tokenizer_path" not in model and "path" in model:
        model["tokenizer_path"] = model["path"]
    conf.setdefault("truncation", None)
    return conf


def patch_from_config(model, conf):
    """``patch_hf`` with the ``model`` section of a loaded configuration, as pred.py:56 calls it."""
    from .patch import patch_hf
    return patch_hf(model, conf.model.type, **conf.model)
