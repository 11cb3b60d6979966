"""Tensor tracing and golden dumps for parity work (interface of sharktank/sharktank/utils/debugging.py:24-122).

Same switches as the reference, read once from the environment variable `TURBINE_LLM_DEBUG`, a comma-separated list of
`name`, `+name`, `-name` or `name=value`:

* `tensor_trace`            print every traced tensor (`::: TRACE key:name(shape, dtype) = ...`)
* `enable_nan_checks`       make `BaseLayer.assert_not_nan` check its arguments
* `save_goldens_path=DIR`   write every golden trace to `DIR/NNNN_key.safetensors`, NNNN counting the dumps in call order

A model that calls `self.trace_tensor("mixtral.moe_block.3.output", h)` on the reference therefore produces the same
stream of records and files here; dumps of the same key from both sides can be compared file by file.  Traced tensors
may live on the GPU: printing and saving copy them to the host, which synchronises, so leave the switches off when
timing.
"""

from __future__ import annotations

import os
import re
import sys
from dataclasses import dataclass
from pathlib import Path
from typing import Dict, Optional

import torch

__all__ = ["DebugFlags", "flags", "trace_tensor", "trace_tensors", "FLAGS_ENV_NAME"]

FLAGS_ENV_NAME = "TURBINE_LLM_DEBUG"

_SETTING = re.compile(r"^(?P<sign>[+-])?(?P<name>[^=]+)(?:=(?P<value>.*))?$")
_UNSAFE_IN_FILE_NAMES = re.compile("[" + re.escape("#~!@$%^&*()[]{}:;\"'") + "]")


@dataclass
class DebugFlags:
    enable_tensor_trace: bool = False
    enable_nan_checks: bool = False
    save_goldens_path: Optional[Path] = None
    golden_sequence_value: int = 0

    def set(self, setting: str) -> None:
        m = _SETTING.match(setting)
        if m is None:
            print(f"{FLAGS_ENV_NAME}: cannot parse '{setting}'", file=sys.stderr)
            return
        on = m.group("sign") != "-"
        name, value = m.group("name"), m.group("value")
        if name == "tensor_trace":
            self.enable_tensor_trace = on
        elif name == "enable_nan_checks":
            self.enable_nan_checks = on
        elif name == "save_goldens_path":
            self.save_goldens_path = Path(value) if (on and value) else None
        elif name == "use_custom_iree_kernels":
            pass  # accepted for compatibility: there is only the HIP path here
        else:
            print(f"{FLAGS_ENV_NAME}: unknown flag '{name}'", file=sys.stderr)

    @staticmethod
    def parse(settings: str) -> "DebugFlags":
        parsed = DebugFlags()
        for piece in settings.split(","):
            piece = piece.strip()
            if piece:
                parsed.set(piece)
        return parsed

    @staticmethod
    def parse_from_env() -> "DebugFlags":
        settings = os.getenv(FLAGS_ENV_NAME)
        return DebugFlags() if settings is None else DebugFlags.parse(settings)


flags = DebugFlags.parse_from_env()


def trace_tensor(key: str, t: Optional[torch.Tensor], *, values: bool = True, golden: bool = False) -> None:
    trace_tensors(key, {"default": t}, values=values, golden=golden)


def trace_tensors(key: str, tensors: Dict[str, Optional[torch.Tensor]], *, values: bool = True, golden: bool = False) -> None:
    if golden:
        if flags.save_goldens_path is not None:
            _save_goldens(key, tensors)
        return
    if not flags.enable_tensor_trace:
        return
    for name, t in tensors.items():
        if t is None:
            continue
        shown = repr(t) if values else "...elided..."
        print(f"::: TRACE {key}:{name}({list(t.shape), t.dtype}) =\n{shown}")


def _save_goldens(key: str, tensors: Dict[str, Optional[torch.Tensor]]) -> None:
    from safetensors.torch import save_file

    sequence = flags.golden_sequence_value
    flags.golden_sequence_value = sequence + 1
    path = Path(flags.save_goldens_path) / f"{sequence:04d}_{_UNSAFE_IN_FILE_NAMES.sub('', key)}.safetensors"
    path.parent.mkdir(parents=True, exist_ok=True)
    print(f"::: SAVE GOLDEN {path}")
    save_file({name: t.detach().contiguous().cpu() for name, t in tensors.items() if t is not None}, str(path))
