"""One registry from an architecture's name (config.json `architectures[0]`, or `architecture`) to
its typed configuration, and through `to_spec()` to its model.  A configuration
class offers `from_dict(config_json) -> cfg`, `cfg.to_dict()`, `cfg.to_spec()
-> ModelSpec` and optionally `cfg.with_window(n)` and `cfg.with_tensor_shapes(shape_of)` (a design that leaves
sizes to the shapes of a folder's tensors: `config_from_folder` calls it with the folder's shapes)."""
import json
import os

from .llama import ConfigError, LlamaConfig
from .bovozen import BovozenConfig
from .gedunex import GedunexConfig
from .rekirax import RekiraxConfig
from .situlorn import SitulornConfig

_ARCHITECTURES = {}


def register_architecture(name, config_class, replace=False):
    if name in _ARCHITECTURES and not replace and _ARCHITECTURES[name] is not config_class:
        raise ValueError("architecture %r is already registered" % name)
    _ARCHITECTURES[name] = config_class


def unregister_architecture(name):
    _ARCHITECTURES.pop(name, None)


def registered_architectures():
    return sorted(_ARCHITECTURES)


def config_from_dict(d):
    """The typed configuration of a config.json dictionary, chosen by its architecture."""
    archs = d.get("architectures") or []
    name = archs[0] if archs else d.get("architecture")
    if name not in _ARCHITECTURES:
        # convert.py:24-27: an unknown architecture is an error that lists the known ones
        raise ConfigError("architecture %r is not supported; registered: %s" % (name, registered_architectures()))
    return _ARCHITECTURES[name].from_dict(d)


def config_from_folder(path):
    f = os.path.join(path, "config.json")
    if not os.path.exists(f):
        raise ConfigError("no config.json in %s" % path)                # convert.py:223-224
    with open(f) as fh:
        cfg = config_from_dict(json.load(fh))
    if hasattr(cfg, "with_tensor_shapes"):
        cfg = cfg.with_tensor_shapes(_folder_shapes(path))
    return cfg


def _folder_shapes(path):
    """name -> shape (or None) over the headers of a folder's *.safetensors files; no tensor is read."""
    from ..weights.safetensors_io import SafetensorsError, SafetensorsFile
    shapes = {}
    for n in sorted(os.listdir(path)):
        if n.endswith(".safetensors"):
            try:
                for key, entry in SafetensorsFile(os.path.join(path, n)).entries.items():
                    shapes[key] = tuple(entry.shape)
            except SafetensorsError:
                pass                        # the loader reports a broken file with its own words
    return shapes.get


for _cls in (LlamaConfig, SitulornConfig, GedunexConfig, BovozenConfig, RekiraxConfig):
    for _name in _cls.ARCHITECTURES:
        register_architecture(_name, _cls)
