"""Stage descriptors and YAML pipelines for the HIP target.

Grammar and file format follow lighthouse/pipeline/descriptor.py:8-287:

    name[arg=val,flag]{opt=val other_flag}

is one stage (``[]`` comma separated arguments, ``{}`` space separated options, values
converted with ``string_to_type``, bare names meaning True), and a pipeline file is

    Pipeline:
      - kernel:  matmul{tile_m=256 tile_n=256 ...}
      - include: other.yaml
      - pass / transform / schedule: ...     (MLIR stages; parsed, not runnable here)

with ``$var`` replaced by the options given to the including descriptor.  A ``kernel`` stage
names the C ABI payload entry point that implements the pipeline on gfx950 and records the
tile parameters the hand-written kernel uses, where the reference's XeGPU descriptor
(lighthouse/pipeline/descriptors/xegpu/matmul/bf16.yaml) records its schedule parameters.
"""

from __future__ import annotations

import os
import re
from dataclasses import dataclass, field

import yaml


def string_to_type(value):
    """Text -> None / bool / int / float / list / tuple / str (lighthouse/utils/types.py:30-80)."""
    if value is None:
        return None
    try:
        value = str(value)
    except Exception:
        return None
    if not value:
        return value
    low = value.lower()
    if low == "none":
        return None
    if low in ("true", "false"):
        return low == "true"
    for conv in (int, float):
        try:
            return conv(value)
        except ValueError:
            pass
    for open_, close, make in (("[", "]", list), ("(", ")", tuple)):
        if value.startswith(open_) and value.endswith(close):
            inner = value[1:-1]
            return make(string_to_type(v.strip()) for v in inner.split(",")) if inner else make()
    return value


_STAGE_TYPES = ("kernel", "pass", "transform", "schedule", "include")


class Descriptor:
    """One stage: basename + ``args`` + ``opts`` (+ its kind and the directory it came from)."""

    def __init__(self, descriptor: str = "", args: dict | None = None, opts: dict | None = None,
                 type: str | None = None, base_path: str | None = None):
        self.type = type
        self.base_path = base_path
        if descriptor and not args and not opts:
            self.basename, self.args, self.opts = self._parse_args_and_opts(descriptor)
        else:
            self.basename = descriptor
            self.args = dict(args or {})
            self.opts = dict(opts or {})
        if self.is_include():
            self.basename = self._resolve_include()
        if self.base_path is None and self.basename:
            self.base_path = os.path.dirname(self.basename)

    # -- classification (explicit type wins; otherwise inferred from the name) --
    def is_kernel(self) -> bool:
        return self.type == "kernel"

    def is_include(self) -> bool:
        if self.type is not None:
            return self.type == "include"
        if self.basename and not self.args and not self.opts and self.basename.endswith(".yaml"):
            self.type = "include"
            return True
        return False

    def is_transform(self) -> bool:
        if self.type is not None:
            return self.type in ("transform", "schedule")
        if self.basename and self.basename.endswith((".mlir", ".py")):
            self.type = "transform"
            return True
        return False

    def is_pass(self) -> bool:
        if self.type is not None:
            return self.type == "pass"
        if self.basename and not self.args and not self.opts and not re.search(r"\.\w+$", self.basename):
            self.type = "pass"
            return True
        return False

    def _resolve_include(self) -> str:
        name = self._strip(self.basename)
        if os.path.exists(os.path.abspath(name)):
            return name
        roots = [self.base_path] if self.base_path else []
        roots.append(os.path.join(os.path.dirname(__file__), "descriptors"))
        for root in roots:
            candidate = os.path.join(root, name)
            if os.path.exists(candidate):
                return candidate
        raise ValueError(f"Included pipeline descriptor file does not exist: {name} (searched in {roots})")

    @staticmethod
    def _parse_csv(text: str, separator: str) -> dict:
        out = {}
        for item in str(text).split(separator):
            if not item:
                continue
            if "=" in item:
                key, value = item.split("=", 1)
                out[key.strip()] = string_to_type(value.strip())
            else:
                out[item.strip()] = True
        return out

    @staticmethod
    def _strip(line: str) -> str:
        m = re.search(r"^([^[{]*)", str(line))
        return m.group(1) if m else str(line)

    @staticmethod
    def _parse_args_and_opts(line: str):
        line = str(line)
        args, opts = {}, {}
        # [] arguments only when the bracket opens before any {} (lists may occur inside options)
        if re.match(r"[^{]+\[", line):
            m = re.search(r"\[([^]]*)\]", line)
            if m:
                args = Descriptor._parse_csv(m.group(1).strip(), ",")
        m = re.search(r"\{([^}]+)\}", line)
        if m:
            opts = Descriptor._parse_csv(" ".join(m.group(1).split()), " ")
        return Descriptor._strip(line).strip(), args, opts

    def __str__(self) -> str:
        args = "[" + ",".join(f"{k}={v}" for k, v in self.args.items()) + "]" if self.args else ""
        opts = ""
        if self.opts:
            opts = "{" + " ".join(k if v is True else f"{k}={v}" for k, v in self.opts.items()) + "}"
        return f"{self.basename}{args}{opts}"


@dataclass
class KernelStage:
    """A resolved ``kernel`` stage: which payload entry point runs and with which parameters."""

    entry: str
    params: dict = field(default_factory=dict)


class PipelineDescriptor:
    """A YAML pipeline file flattened (includes expanded, variables substituted) into stages."""

    def __init__(self, desc: Descriptor):
        if not isinstance(desc, Descriptor):
            raise ValueError(f"PipelineDescriptor requires a Descriptor as input, got {type(desc)}")
        self.descriptor = desc
        self.base_path = os.path.dirname(desc.basename) if desc.basename else desc.base_path
        with open(desc.basename) as f:
            self.pipeline_desc = yaml.safe_load(f) or {}
        self.stages: list[Descriptor] = []
        entries = self.pipeline_desc.get("Pipeline") or []
        for item in entries:
            key, line = next(iter(item.items()))
            if key not in _STAGE_TYPES:
                raise ValueError(f"Invalid stage in pipeline description: {key}: {line}.")
            line = str(line)
            for var, value in desc.opts.items():
                line = line.replace("$" + var, str(value).replace(" ", ""))
            stage = Descriptor(line, type=key, base_path=self.base_path)
            if stage.is_include():
                self.stages.extend(PipelineDescriptor(stage).get_stages())
            else:
                self.stages.append(stage)
        if not self.stages:
            raise ValueError(f"Pipeline description file {desc.basename} does not contain a valid 'Pipeline'.")

    def get_stages(self) -> list[Descriptor]:
        return self.stages

    def kernel_stages(self) -> list[KernelStage]:
        return [KernelStage(s.basename, {**s.args, **s.opts}) for s in self.stages if s.is_kernel()]

    def unsupported_stages(self) -> list[Descriptor]:
        """MLIR pass / transform stages: they need the MLIR bindings and cannot run on this target."""
        return [s for s in self.stages if not s.is_kernel()]
