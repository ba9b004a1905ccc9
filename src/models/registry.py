"""
Model-class registry: which model class serves a checkpoint directory, decided by its ``config.json``.

* HuggingFace-format Llama / Mistral / Mixtral (``model_type``) -> :class:`src.models.llama.CausalLM`;
* ``"architecture": "Datatar"`` (layers listed in the config) -> :class:`src.models.datatar.DatatarLM`;
* ``"architecture": "Fekolorn"`` (layers listed in the config, per-sequence state) ->
  :class:`src.models.fekolorn.FekolornLM`;
* ``"architecture": "Bapivik"`` (layers listed in the config, learned positions, depth-averaged layer results) ->
  :class:`src.models.bapivik.BapivikLM`;
* ``"architecture": "Kogerax"`` (layers listed in the config: matrix-memory LSTM, scalar-decay state space, attention
  beside a selective scan; unnormed sublayer inputs, normed outputs) -> :class:`src.models.kogerax.KogeraxLM`.

A new family registers a (matcher, arch reader, model class) triple with :func:`register_family`.
"""

from __future__ import annotations

import json
import os
from typing import Callable, Dict, List, Tuple

_FAMILIES: List[Tuple[str, Callable[[dict], bool], Callable, Callable]] = []


def register_family(name: str, matches: Callable[[dict], bool], read_arch: Callable, model_class: Callable) -> None:
    """matches(config dict) -> bool; read_arch(path, **overrides) -> arch; model_class() -> the class (lazy)."""
    _FAMILIES.append((name, matches, read_arch, model_class))


def _read_config(path: str) -> dict:
    with open(os.path.join(path, "config.json")) as f:
        return json.load(f)


def family_of(path: str) -> str:
    c = _read_config(path)
    for name, matches, _, _ in _FAMILIES:
        if matches(c):
            return name
    raise ValueError(f"{path}: no registered model family matches config.json "
                     f"(architecture={c.get('architecture')!r}, model_type={c.get('model_type')!r})")


def resolve(path: str, **arch_overrides):
    """(family name, arch, model class) of a checkpoint directory."""
    c = _read_config(path)
    for name, matches, read_arch, model_class in _FAMILIES:
        if matches(c):
            return name, read_arch(path, **arch_overrides), model_class()
    raise ValueError(f"{path}: no registered model family matches config.json "
                     f"(architecture={c.get('architecture')!r}, model_type={c.get('model_type')!r})")


def families() -> Dict[str, Callable]:
    return {name: cls for name, _, _, cls in _FAMILIES}


def _llama_cls():
    from src.models.llama import CausalLM

    return CausalLM


def _llama_arch(path: str, **kw):
    from src.models.loader import arch_from_hf_config

    return arch_from_hf_config(path, **kw)


def _datatar_cls():
    from src.models.datatar import DatatarLM

    return DatatarLM


def _datatar_arch(path: str, **kw):
    from src.models.datatar import datatar_arch_from_dir

    return datatar_arch_from_dir(path, **kw)


def _fekolorn_cls():
    from src.models.fekolorn import FekolornLM

    return FekolornLM


def _fekolorn_arch(path: str, **kw):
    from src.models.fekolorn import fekolorn_arch_from_dir

    return fekolorn_arch_from_dir(path, **kw)


def _bapivik_cls():
    from src.models.bapivik import BapivikLM

    return BapivikLM


def _bapivik_arch(path: str, **kw):
    from src.models.bapivik import bapivik_arch_from_dir

    return bapivik_arch_from_dir(path, **kw)


def _kogerax_cls():
    from src.models.kogerax import KogeraxLM

    return KogeraxLM


def _kogerax_arch(path: str, **kw):
    from src.models.kogerax import kogerax_arch_from_dir

    return kogerax_arch_from_dir(path, **kw)


register_family("datatar", lambda c: c.get("architecture") == "Datatar", _datatar_arch, _datatar_cls)
register_family("fekolorn", lambda c: c.get("architecture") == "Fekolorn", _fekolorn_arch, _fekolorn_cls)
register_family("bapivik", lambda c: c.get("architecture") == "Bapivik", _bapivik_arch, _bapivik_cls)
register_family("kogerax", lambda c: c.get("architecture") == "Kogerax", _kogerax_arch, _kogerax_cls)
register_family("llama", lambda c: "architecture" not in c and c.get("model_type", "llama") in
                ("llama", "mistral", "mixtral"), _llama_arch, _llama_cls)
