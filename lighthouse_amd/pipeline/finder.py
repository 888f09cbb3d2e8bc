"""Descriptor lookup by target.

Same search as lighthouse/pipeline/finder.py:12-92: ``<base>/<arch>/<feature>/<pipeline>/
<dtype>.yaml`` for every feature the target has, then ``<base>/<arch>/<pipeline>/<dtype>.yaml``;
an external ``base_path`` is searched before the packaged descriptors.  The HIP target is the
directory ``descriptors/gfx950`` the way the reference's Intel target is ``descriptors/xegpu``.
"""

from __future__ import annotations

import os
from pathlib import Path

from ..execution.target import TargetInfo

# Directory holding the pipeline descriptors packaged with this runtime.
DESCRIPTORS_REPO = Path(__file__).parent / "descriptors"


def find_pipeline_file(
    target: TargetInfo | None,
    pipeline: str,
    dtype: str = "f32",
    base_path: str | None = None,
) -> tuple[str | None, str | None]:
    """(path, feature) of the descriptor for ``pipeline``/``dtype`` on ``target``, or (None, None)."""
    if not pipeline or not target:
        return None, None
    if base_path is not None:
        file, feature = _find_pipeline_in_base(target, base_path, pipeline, dtype)
        if file is not None:
            return file, feature
    return _find_pipeline_in_base(target, DESCRIPTORS_REPO, pipeline, dtype)


def _find_pipeline_in_base(target: TargetInfo, base_path, pipeline: str, dtype: str):
    base_path = Path(base_path)
    if not base_path.exists() or not (base_path / target.arch).exists():
        return None, None
    arch_path = base_path / target.arch
    available = [name for name in os.listdir(arch_path) if (arch_path / name).is_dir()]
    for feature in target.has_features(available):
        candidate = arch_path / feature / pipeline / f"{dtype}.yaml"
        if candidate.exists():
            return str(candidate), feature
    if target.arch:
        candidate = arch_path / pipeline / f"{dtype}.yaml"
        if candidate.exists():
            return str(candidate), None
    return None, None
