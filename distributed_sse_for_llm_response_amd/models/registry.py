"""Model registry: one place that maps a model name or a checkpoint directory to its family -- configuration class,
weight loading into the engine's layout, and the runner that holds its forward passes.

A family is chosen by name (``mistral-7b-v0.3``, ``muderax-tiny``, ...) or, for a directory, by the ``architecture`` /
``architectures`` entry of its ``config.json``.  The serving launcher, the benchmark harness and the trace replayer all
come through ``resolve`` / ``load_weights`` / ``make_runner``, so a new family is added here and nowhere else.
"""
from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path

import torch


@dataclass(frozen=True)
class Family:
    name: str
    architectures: tuple      # config.json architecture names that select it
    config_from_dict: object  # (dict, name) -> config
    named: dict               # {config name: config}
    random_weights: object    # (cfg, device, dtype, seed, tp_rank, tp_size) -> engine weights
    load_dir: object          # (cfg, path, device, dtype, tp_rank, tp_size) -> engine weights
    runner: object            # () -> runner class
    dtypes: tuple             # element types its kernels run in


def _mistral() -> Family:
    from . import mistral as M

    def from_dict(d: dict, name: str):
        return M.MistralConfig(name=name, vocab_size=d["vocab_size"], hidden_size=d["hidden_size"],
                               intermediate_size=d["intermediate_size"], num_layers=d["num_hidden_layers"],
                               num_heads=d["num_attention_heads"], num_kv_heads=d.get("num_key_value_heads",
                                                                                      d["num_attention_heads"]),
                               head_dim=d.get("head_dim", d["hidden_size"] // d["num_attention_heads"]),
                               rope_theta=d.get("rope_theta", 10000.0), rms_eps=d.get("rms_norm_eps", 1e-5),
                               max_position=d.get("max_position_embeddings", 32768),
                               bos_token_id=d.get("bos_token_id", 1), eos_token_id=d.get("eos_token_id", 2))

    def random_weights(cfg, device, dtype, seed, tp_rank, tp_size):
        from ..engine import weights as W

        if torch.device(device).type == "cuda":
            return W.random_engine_weights(cfg, tp_rank=tp_rank, tp_size=tp_size, device=device, seed=seed)
        return W.convert_standard(cfg, M.init_standard_weights(cfg, seed=seed), tp_rank=tp_rank, tp_size=tp_size)

    def load_dir(cfg, path, device, dtype, tp_rank, tp_size):
        from ..engine.weights import load_safetensors

        return load_safetensors(cfg, path, tp_rank, tp_size, device)

    def runner():
        from ..engine.model_runner import ModelRunner

        return ModelRunner

    return Family("mistral", ("MistralForCausalLM", "LlamaForCausalLM"), from_dict, dict(M.CONFIGS), random_weights,
                  load_dir, runner, (torch.bfloat16,))


def _muderax() -> Family:
    from . import muderax as X

    def random_weights(cfg, device, dtype, seed, tp_rank, tp_size):
        from ..engine.weights import convert_layered

        cfg.validate(tp_size)
        return convert_layered(cfg, X.init_weights(cfg, seed=seed, device=device), device=device, dtype=dtype)

    def load_dir(cfg, path, device, dtype, tp_rank, tp_size):
        from ..engine.weights import load_layered_dir

        cfg.validate(tp_size)
        return load_layered_dir(cfg, path, device=device, dtype=dtype)

    def runner():
        from ..engine.layered_runner import LayeredRunner

        return LayeredRunner

    return Family("muderax", ("Muderax",), X.MuderaxConfig.from_dict, dict(X.CONFIGS), random_weights, load_dir, runner,
                  (torch.bfloat16, torch.float32))


def _surodra() -> Family:
    from . import surodra as S

    def random_weights(cfg, device, dtype, seed, tp_rank, tp_size):
        from ..engine.weights import convert_surodra

        cfg.validate(tp_size)
        return convert_surodra(cfg, S.init_weights(cfg, seed=seed, device=device), device=device, dtype=dtype)

    def load_dir(cfg, path, device, dtype, tp_rank, tp_size):
        from ..engine.weights import load_surodra_dir

        cfg.validate(tp_size)
        return load_surodra_dir(cfg, path, device=device, dtype=dtype)

    def runner():
        from ..engine.layered_runner import LayeredRunner

        return LayeredRunner

    return Family("surodra", ("Surodra",), S.SurodraConfig.from_dict, dict(S.CONFIGS), random_weights, load_dir, runner,
                  (torch.bfloat16, torch.float32))


def _dironex() -> Family:
    from . import dironex as D

    def random_weights(cfg, device, dtype, seed, tp_rank, tp_size):
        from ..engine.weights import convert_dironex

        cfg.validate(tp_size)
        return convert_dironex(cfg, D.init_weights(cfg, seed=seed, device=device), device=device, dtype=dtype)

    def load_dir(cfg, path, device, dtype, tp_rank, tp_size):
        from ..engine.weights import load_dironex_dir

        cfg.validate(tp_size)
        return load_dironex_dir(cfg, path, device=device, dtype=dtype)

    def runner():
        from ..engine.layered_runner import LayeredRunner

        return LayeredRunner

    return Family("dironex", ("Dironex",), D.DironexConfig.from_dict, dict(D.CONFIGS), random_weights, load_dir, runner,
                  (torch.bfloat16, torch.float32))


def _murulorn() -> Family:
    from . import murulorn as U

    def random_weights(cfg, device, dtype, seed, tp_rank, tp_size):
        from ..engine.weights import convert_murulorn

        cfg.validate(tp_size)
        return convert_murulorn(cfg, U.init_weights(cfg, seed=seed, device=device), device=device, dtype=dtype)

    def load_dir(cfg, path, device, dtype, tp_rank, tp_size):
        from ..engine.weights import load_murulorn_dir

        cfg.validate(tp_size)
        return load_murulorn_dir(cfg, path, device=device, dtype=dtype)

    def runner():
        from ..engine.layered_runner import LayeredRunner

        return LayeredRunner

    return Family("murulorn", ("Murulorn",), U.MurulornConfig.from_dict, dict(U.CONFIGS), random_weights, load_dir, runner,
                  (torch.bfloat16, torch.float32))


_FAMILIES = None


def families() -> dict:
    global _FAMILIES
    if _FAMILIES is None:
        _FAMILIES = {f.name: f for f in (_mistral(), _muderax(), _surodra(), _dironex(), _murulorn())}
    return _FAMILIES


def resolve(model: str):
    """(family, config, checkpoint directory or None) for a config name or a directory with ``config.json``."""
    p = Path(model)
    if p.is_dir() and (p / "config.json").exists():
        d = json.loads((p / "config.json").read_text())
        archs = d.get("architectures") or [d.get("architecture")]
        for fam in families().values():
            if any(a in fam.architectures for a in archs):
                return fam, fam.config_from_dict(d, p.name), str(p)
        raise ValueError(f"{p}/config.json names no known architecture ({archs}); known: "
                         f"{sorted(a for f in families().values() for a in f.architectures)}")
    for fam in families().values():
        if model in fam.named:
            return fam, fam.named[model], None
    names = sorted(n for f in families().values() for n in f.named)
    raise ValueError(f"unknown model {model!r}: neither a checkpoint directory nor one of {names}")


def family_of(cfg) -> Family:
    return families()[getattr(cfg, "family", "mistral")]


def load_weights(fam: Family, cfg, path=None, device="cpu", dtype=torch.bfloat16, seed: int = 0, tp_rank: int = 0,
                 tp_size: int = 1):
    """Engine weights of `cfg`: from the checkpoint directory `path`, else random from `seed`."""
    if dtype not in fam.dtypes:
        raise ValueError(f"the {fam.name} family runs in {[str(t) for t in fam.dtypes]}, not {dtype}")
    if path:
        return fam.load_dir(cfg, path, device, dtype, tp_rank, tp_size)
    return fam.random_weights(cfg, device, dtype, seed, tp_rank, tp_size)


def make_runner(fam: Family, weights, **kw):
    return fam.runner()(weights, **kw)


def cache_blocks_for_budget(cfg, budget_bytes: int, tp_size: int = 1, elem_bytes: int = 2) -> int:
    """Pages of the family's cache that fit `budget_bytes`."""
    from ..engine.kv_cache import PAGE, KVCache

    if getattr(cfg, "family", "mistral") in ("muderax", "surodra", "dironex", "murulorn"):
        return max(1, budget_bytes // max(1, cfg.cache_bytes_per_token(elem_bytes) * PAGE))
    return KVCache.blocks_for_budget(budget_bytes, cfg.num_layers, cfg.num_kv_heads // tp_size)
