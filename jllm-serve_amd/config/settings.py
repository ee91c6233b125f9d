"""Layered settings in the reference's manner (config/Settings.java:31-75, :88-127, :156-202, :212-355):
bundled defaults < external properties file < command-line flags; short aliases for common keys; an unknown
key is an error; every typed value is parsed once, before any weight is loaded."""
from __future__ import annotations

import os
from typing import Dict, List, Optional, Tuple

RESOURCE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "jllm.properties")

# short flag -> property key (config/Settings.java:31-75, the ones this engine has)
ALIASES = {
    "model": "model.repo", "dir": "model.dir", "dtype": "backend.dtype", "ctx": "backend.ctx", "batch": "backend.batch",
    "temp": "sampling.temperature", "temperature": "sampling.temperature", "top-k": "sampling.top-k",
    "top-p": "sampling.top-p", "min-p": "sampling.min-p", "rep-penalty": "sampling.repetition-penalty",
    "seed": "sampling.seed", "max-tokens": "sampling.max-tokens", "page-size": "backend.kv-block",
    "slots": "server.slots",
}
# per-invocation inputs that are not properties (config/Settings.java:77-79)
CLI_ONLY = {"prompt", "raw", "config", "ignore-eos", "random-weights", "config-json", "out", "json"}
BOOLEAN_KEYS = {"raw", "ignore-eos", "json"}
_BOOL = {"true": True, "yes": True, "on": True, "1": True, "false": False, "no": False, "off": False, "0": False}


class SettingsError(ValueError):
    pass


def read_properties(path: str) -> Dict[str, str]:
    out: Dict[str, str] = {}
    with open(path, "r", encoding="utf-8") as f:
        for line in f:
            line = line.strip()
            if not line or line[0] in "#!":
                continue
            if "=" not in line:
                raise SettingsError(f"{path}: expected key=value, got '{line}'")
            k, v = line.split("=", 1)
            out[k.strip()] = v.strip()
    return out


def parse_args(args: List[str]) -> Dict[str, str]:
    """``--key value``, ``--key=value`` or, for a boolean key, a bare ``--flag`` that consumes the next argument
    only when it is a boolean literal; a stray positional argument after the command word is an error."""
    m: Dict[str, str] = {}
    i = 0
    while i < len(args):
        a = args[i]
        if not a.startswith("--"):
            if i == 0:
                i += 1
                continue  # the command word
            raise SettingsError(f"unexpected argument '{a}' (options are --key value or --key=value; boolean flags "
                                "take true/false or stand alone)")
        key = a[2:]
        if "=" in key:
            key, value = key.split("=", 1)
        else:
            key = ALIASES.get(key, key)
            nxt = args[i + 1] if i + 1 < len(args) else None
            if nxt is None or nxt.startswith("--"):
                value = "true"
            elif key in BOOLEAN_KEYS and nxt.lower() not in _BOOL:
                value = "true"
            else:
                value = nxt
                i += 1
        m[ALIASES.get(key, key)] = value
        i += 1
    return m


class Settings:
    def __init__(self):
        self.props: Dict[str, str] = {}
        self.sources: Dict[str, str] = {}

    @classmethod
    def load(cls, args: List[str], env=None) -> "Settings":
        env = os.environ if env is None else env
        s = cls()
        for k, v in read_properties(RESOURCE).items():
            s.props[k] = v
            s.sources[k] = "default"
        flags = parse_args(args)
        external = flags.get("config") or env.get("JLLM_CONFIG") or ("jllm.properties" if os.path.exists("jllm.properties") else None)
        if external:
            if not os.path.exists(external):
                raise SettingsError(f"config file not found: {external}")
            for k, v in read_properties(external).items():
                s._put(k, v, external)
        for k, v in flags.items():
            s._put(k, v, "flag")
        return s

    def _put(self, key: str, value: str, source: str) -> None:
        if key not in self.props and key not in CLI_ONLY:
            raise SettingsError(f"unknown option --{key} (see jllm.properties for valid keys)")
        self.props[key] = value.strip()
        self.sources[key] = source

    def has(self, key: str) -> bool:
        return key in self.props and self.props[key] != ""

    def get(self, key: str) -> str:
        return self.props[key]

    def get_int(self, key: str) -> int:
        try:
            return int(self.props[key])
        except ValueError:
            raise SettingsError(f"{key} must be an integer, got '{self.props[key]}'") from None

    def get_float(self, key: str) -> float:
        try:
            return float(self.props[key])
        except ValueError:
            raise SettingsError(f"{key} must be a number, got '{self.props[key]}'") from None

    def get_bool(self, key: str) -> bool:
        v = self.props.get(key, "false").lower()
        if v not in _BOOL:
            raise SettingsError(f"{key} must be true or false, got '{self.props[key]}'")
        return _BOOL[v]

    def int_or_auto(self, key: str) -> Optional[int]:
        return None if self.props[key].lower() == "auto" else self.get_int(key)

    def validate(self) -> "Settings":
        """Parses every typed setting once so that a typo fails before the weights load (Settings.java:212-355)."""
        if self.get("backend.dtype").lower() not in ("bfloat16", "bf16", "float32", "fp32", "f32"):
            raise SettingsError(f"backend.dtype must be bfloat16 or float32, got '{self.get('backend.dtype')}'")
        for k in ("backend.ctx", "backend.batch"):
            v = self.int_or_auto(k)
            if v is not None and v < 1:
                raise SettingsError(f"{k} must be auto or a positive integer, got {v}")
        self.get_bool("backend.kv-prefix-share")
        self.get_bool("engine.preempt")
        b = self.get_int("backend.kv-block")
        if b < 1 or b & (b - 1):
            raise SettingsError(f"backend.kv-block must be a power of two, got {b}")
        for k in ("backend.kv-pool-tokens", "backend.ctx-max", "engine.pass-budget", "engine.mixed-reserve",
                  "engine.max-running", "engine.background-chunk-cap", "engine.age-promote-ms", "engine.session-max-running", "bench.max-tokens", "bench.rounds", "bench.prompt-repeat"):
            if self.get_int(k) < 0:
                raise SettingsError(f"{k} must not be negative")
        if self.get_int("server.slots") < 1:
            raise SettingsError("server.slots must be at least 1")
        self.sampling()
        return self

    def sampling(self):
        from ..sampling.params import SamplingParams
        try:
            return SamplingParams(
                temperature=self.get_float("sampling.temperature"), top_k=self.get_int("sampling.top-k"),
                top_p=self.get_float("sampling.top-p"), min_p=self.get_float("sampling.min-p"),
                repetition_penalty=self.get_float("sampling.repetition-penalty"),
                presence_penalty=self.get_float("sampling.presence-penalty"),
                frequency_penalty=self.get_float("sampling.frequency-penalty"), seed=self.get_int("sampling.seed"),
                max_tokens=self.get_int("sampling.max-tokens"), ignore_eos=self.get_bool("ignore-eos"))
        except ValueError as e:
            raise SettingsError(str(e)) from None

    def describe(self) -> List[Tuple[str, str, str]]:
        return [(k, self.props[k], self.sources.get(k, "default")) for k in sorted(self.props)]
