"""Model registry: which engine serves a model folder, decided by its config.json.

Hugging Face style configurations name their family in ``model_type`` / ``architectures`` (Qwen3, Qwen3.5); Duguzen,
Feruzen, Ramalix and Kukulorn name it in ``architecture``.  ``load_engine`` builds the engine with the weights of the folder; ``scheduler_for`` puts the
continuous-batching scheduler (include/pegainfer_scheduler.h) on top of it.
"""
import json
import os


def _qwen3(model_dir, cfg, **kw):
    from .qwen3 import Qwen3Engine
    pages = max(2, (kw.get("max_tokens", 4096) + 15) // 16 + 1)
    eng = Qwen3Engine(cfg, num_kv_pages=pages, max_batch_size=kw.get("max_requests", 8), device=kw.get("device", 0))
    return eng.load_safetensors(os.path.join(model_dir, "model.safetensors"))


def _qwen35(model_dir, cfg, **kw):
    from .qwen35 import Qwen35Engine
    cfg = cfg.get("text_config", cfg)
    pages = max(2, (kw.get("max_tokens", 4096) + 15) // 16 + 1)
    eng = Qwen35Engine(cfg, num_kv_pages=pages, max_batch_size=kw.get("max_requests", 8), device=kw.get("device", 0))
    return eng.load_safetensors(os.path.join(model_dir, "model.safetensors"))


def _duguzen(model_dir, cfg, **kw):
    from .duguzen import DuguzenEngine
    return DuguzenEngine.from_pretrained(model_dir, max_tokens=kw.get("max_tokens", 4096), max_requests=kw.get("max_requests", 8),
                                         dtype=kw.get("dtype", "bfloat16"), device=kw.get("device", 0))


def _feruzen(model_dir, cfg, **kw):
    from .feruzen import FeruzenEngine
    return FeruzenEngine.from_pretrained(model_dir, max_tokens=kw.get("max_tokens", 4096), max_requests=kw.get("max_requests", 8),
                                         dtype=kw.get("dtype", "bfloat16"), device=kw.get("device", 0))


def _ramalix(model_dir, cfg, **kw):
    from .ramalix import RamalixEngine
    return RamalixEngine.from_pretrained(model_dir, max_tokens=kw.get("max_tokens", 4096), max_requests=kw.get("max_requests", 8),
                                         dtype=kw.get("dtype", "bfloat16"), device=kw.get("device", 0))


def _kukulorn(model_dir, cfg, **kw):
    from .kukulorn import KukulornEngine
    return KukulornEngine.from_pretrained(model_dir, max_tokens=kw.get("max_tokens", 4096), max_requests=kw.get("max_requests", 8),
                                          dtype=kw.get("dtype", "bfloat16"), device=kw.get("device", 0))


# family -> (loader, dtypes it can be served in)
REGISTRY = {
    "qwen3": (_qwen3, ("bfloat16",)),
    "qwen3_5": (_qwen35, ("bfloat16",)),
    "duguzen": (_duguzen, ("bfloat16", "float32")),
    "feruzen": (_feruzen, ("bfloat16", "float32")),
    "ramalix": (_ramalix, ("bfloat16", "float32")),
    "kukulorn": (_kukulorn, ("bfloat16", "float32")),
}


def family_of(cfg):
    """the registry key of a parsed config.json, or None"""
    if str(cfg.get("architecture", "")).lower() in ("duguzen", "feruzen", "ramalix", "kukulorn"):
        return str(cfg["architecture"]).lower()
    names = [str(cfg.get("model_type", ""))] + [str(a) for a in cfg.get("architectures", [])]
    low = " ".join(names).lower()
    if "qwen3_5" in low or "qwen3.5" in low or "qwen35" in low or "linear_num_key_heads" in cfg.get("text_config", cfg):
        return "qwen3_5"
    if "qwen3" in low:
        return "qwen3"
    return None


def read_config(model_dir):
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def load_engine(model_dir, dtype="bfloat16", **kw):
    cfg = read_config(model_dir)
    fam = family_of(cfg)
    if fam is None:
        raise ValueError("no engine is registered for the model in " + model_dir)
    loader, dtypes = REGISTRY[fam]
    if dtype not in dtypes:
        raise ValueError("%s is served in %s only" % (fam, " / ".join(dtypes)))
    return loader(model_dir, cfg, dtype=dtype, **kw)


def scheduler_for(engine, seed=42, stop_tokens=()):
    from .scheduler import Scheduler
    return Scheduler.over_engine(engine, seed=seed, stop_tokens=stop_tokens)
