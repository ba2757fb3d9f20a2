"""Engine options: generation defaults, scheduler limits, cache sizing.

Option names and meanings are the reference's YAML ones
(src/qwen3_from_scratch/factory/batch_config.py:83-164,235-334): a `generation`
block, a `scheduler` block, per-model `path`/`dtype`/`max_len`. The same YAML
file is accepted by `EngineConfig.from_yaml`; keyword arguments work as well.
"""

import dataclasses
import os
from dataclasses import dataclass, field

from .model_config import ConfigError

_DTYPE_ALIASES = {
    "bf16": "bfloat16",
    "bfloat16": "bfloat16",
    "fp32": "float32",
    "float32": "float32",
    "float": "float32",
}


def parse_dtype(value):
    """'bf16', 'bfloat16', 'fp32', 'float32' or 'float' -> 'bfloat16' | 'float32'.

    The reference also lists float16 (batch_config.py:38-47); this engine keeps
    weights in bfloat16 and refuses it.
    """
    key = str(value).replace("torch.", "").strip().lower()
    if key not in _DTYPE_ALIASES:
        raise ConfigError(
            "unsupported dtype %r; valid: %s" % (value, ", ".join(sorted(_DTYPE_ALIASES)))
        )
    return _DTYPE_ALIASES[key]


@dataclass
class GenerationDefaults:
    """Sampling defaults (batch_config.py:83-91). `temperature <= 0` is greedy,
    `top_k > 0` restricts sampling to the k best logits
    (src/qwen3_from_scratch/inference/model_worker.py:32-41). `top_p` and
    `do_sample` are read for compatibility and, as in the reference, unused."""

    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    do_sample: bool = False
    max_new_tokens: int = 100


@dataclass
class EngineConfig:
    path: str = ""
    name: str = ""
    device: str = "cuda"
    dtype: str = "bfloat16"
    max_len: int = 2048
    generation: GenerationDefaults = field(default_factory=GenerationDefaults)
    # scheduler block (batch_config.py:142-149)
    max_num_seqs: int = 32
    max_num_tokens: int = 3000
    block_size: int = 16
    gpu_utilization: float = 0.5
    chunked_prefill_size: int = 512
    # requests take over the cached blocks of a prefix they share with earlier ones (batch_config.py:147)
    enable_prefix_cache: bool = True
    # an explicit number of cache pages; overrides gpu_utilization when set
    num_blocks: int = 0
    seed: int = 0
    use_graphs: bool = True
    # launch a decode step before the previous step's tokens have reached the host
    lookahead: bool = True
    # keep a second copy of every bfloat16 matrix in the order the few-row product kernel streams it:
    # decoding is about a fifth faster with it, and the matrices take their memory twice
    tiled_weights: bool = True
    # other registered implementations for some kinds of parts: {slot: name, or {name, kwargs}}
    # (batch_config.py:209-229); checked here, applied when the model is built
    components: dict = field(default_factory=dict)
    # the reference's option for the cache's dtype (batch_config.py:164,275). The cache here is kept
    # in the compute dtype; any other value is refused rather than ignored. None: not given.
    kv_cache_dtype: str = None
    # further tokens that end a request, beside those the model folder names
    eos_ids: tuple = ()

    def __post_init__(self):
        from .registry import resolve_components

        self.dtype = parse_dtype(self.dtype)
        self.components = dict(self.components or {})
        resolve_components(self.components)           # fails here, not when the model is built
        if self.kv_cache_dtype is not None:
            self.kv_cache_dtype = parse_dtype(self.kv_cache_dtype)
            if self.kv_cache_dtype != self.dtype:
                raise ConfigError(
                    "kv_cache_dtype %s differs from dtype %s: this engine keeps the cache in the compute dtype "
                    "(leave kv_cache_dtype out, or set it to the model's dtype)" % (self.kv_cache_dtype, self.dtype))
        self.eos_ids = tuple(int(t) for t in (self.eos_ids or ()))
        if any(t < 0 for t in self.eos_ids):
            raise ConfigError("eos_ids must be token ids, found %r" % (self.eos_ids,))
        if self.max_len <= 0:
            raise ConfigError("max_len must be positive, found %d" % self.max_len)
        if self.block_size <= 0:
            raise ConfigError("block_size must be positive, found %d" % self.block_size)
        if self.max_num_seqs <= 0 or self.max_num_tokens <= 0:
            raise ConfigError("max_num_seqs and max_num_tokens must be positive")
        if self.chunked_prefill_size <= 0:
            raise ConfigError("chunked_prefill_size must be positive")
        if not (0.0 < self.gpu_utilization <= 1.0):
            raise ConfigError("gpu_utilization must be in (0, 1]")

    @classmethod
    def from_yaml(cls, config_path, model_name, **overrides):
        """Read the reference's YAML layout and pick `model_name` from `models`.

        Per-model `generation` entries override the global block field by field
        (batch_config.py:194-207). A model's `components` are checked against
        the part registry and a top-level `kv_cache_dtype` against the model's
        dtype; what this engine cannot honour is an error, as in the reference
        (batch_config.py:369-382).
        """
        import yaml

        with open(config_path, encoding="utf-8") as fh:
            raw = yaml.safe_load(fh)
        if raw is None:
            raise ConfigError("configuration file is empty: %s" % config_path)
        models = raw.get("models") or []
        if not isinstance(models, list) or not models:
            raise ConfigError("'models' must be a non-empty list")
        names = [m.get("name") for m in models if isinstance(m, dict)]
        if len(set(names)) != len(names):
            raise ConfigError("model names are not unique: %s" % names)
        entry = None
        for m in models:
            if not isinstance(m, dict) or "name" not in m or "path" not in m:
                raise ConfigError("every entry of 'models' needs 'name' and 'path'")
            if m["name"] == model_name:
                entry = m
        if entry is None:
            raise KeyError("model %r is not in %s; available: %s" % (model_name, config_path, names))
        if not os.path.isfile(os.path.join(entry["path"], "config.json")):
            raise ConfigError("model %s: no config.json in %s" % (model_name, entry["path"]))
        gen = dict(raw.get("generation") or {})
        gen.update({k: v for k, v in (entry.get("generation") or {}).items() if v is not None})
        known = {f.name for f in dataclasses.fields(GenerationDefaults)}
        generation = GenerationDefaults(**{k: v for k, v in gen.items() if k in known})
        sched = raw.get("scheduler") or {}
        kwargs = dict(
            path=entry["path"],
            name=entry["name"],
            device=entry.get("device", "cuda"),
            dtype=entry.get("dtype", "bfloat16"),
            max_len=entry.get("max_len", 2048),
            generation=generation,
            components=entry.get("components") or {},
        )
        if "kv_cache_dtype" in raw:
            kwargs["kv_cache_dtype"] = raw["kv_cache_dtype"]
        for key in ("max_num_seqs", "max_num_tokens", "block_size", "gpu_utilization",
                    "chunked_prefill_size", "num_blocks", "enable_prefix_cache"):
            if key in sched:
                kwargs[key] = sched[key]
        kwargs.update(overrides)
        return cls(**kwargs)
