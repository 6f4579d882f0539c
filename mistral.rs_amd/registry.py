"""Model registry: which loader serves a checkpoint.  A folder with `config.json` is dispatched on its `"architecture"`; a `.gguf` file on `general.architecture`
(role of the reference's loader selection, mistralrs-core/src/pipeline/loaders/normal_loaders.rs `NormalLoaderType` + `auto` detection from config.json)."""
from __future__ import annotations

import json
import os
from typing import Callable, Dict

ARCHITECTURES: Dict[str, Callable] = {}


def register(name: str):
    def deco(fn):
        ARCHITECTURES[name] = fn
        return fn
    return deco


@register("Gekilix")
def _load_gekilix(path: str, device, dtype: str = "bfloat16", **kw):
    from .hybrid import HybridDecoder
    return HybridDecoder.from_pretrained(path, device, dtype, **kw)


@register("Sobunex")
def _load_sobunex(path: str, device, dtype: str = "bfloat16", **kw):
    from .hybrid import HybridDecoder
    return HybridDecoder.from_pretrained(path, device, dtype, **kw)


@register("Setopel")
def _load_setopel(path: str, device, dtype: str = "bfloat16", **kw):
    from .hybrid import HybridDecoder
    return HybridDecoder.from_pretrained(path, device, dtype, **kw)


@register("Gifopel")
def _load_gifopel(path: str, device, dtype: str = "bfloat16", **kw):
    from .hybrid import HybridDecoder
    return HybridDecoder.from_pretrained(path, device, dtype, **kw)


@register("llama")
def _load_llama_gguf(path: str, device, dtype: str = "bfloat16", **kw):
    from .gguf.archive import load_llama
    return load_llama(path, device, **kw)


def architecture_of(path: str) -> str:
    if os.path.isdir(path):
        with open(os.path.join(path, "config.json")) as f:
            return json.load(f)["architecture"]
    from .gguf.archive import GgufArchive
    with GgufArchive(path) as a:
        return a.metadata["general.architecture"]


def load_model(path: str, device, dtype: str = "bfloat16", **kw):
    """The model object for a checkpoint (a folder with config.json + model.safetensors, or a GGUF file).  `kw` goes to the architecture's loader (cache sizes)."""
    arch = architecture_of(path)
    if arch not in ARCHITECTURES and arch == "mistral":
        arch = "llama"
    if arch not in ARCHITECTURES:
        raise ValueError(f"no loader registered for architecture {arch!r} (known: {sorted(ARCHITECTURES)})")
    return ARCHITECTURES[arch](path, device, dtype, **kw)
