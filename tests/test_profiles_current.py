"""The summaries under profiles/ must describe the kernels that ship: each one names the commit it was
measured on and the source files of the kernels it profiles, and no later commit may have touched
those files.  (Skipped where the tree has no git history, e.g. on an exported copy.)"""

import json
import re
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
PROFILES = ROOT / "profiles"


def _git(*args):
    return subprocess.run(["git", *args], cwd=ROOT, capture_output=True, text=True)


def _entries():
    out = []
    for path in sorted(PROFILES.iterdir()):
        if path.suffix == ".json":
            d = json.loads(path.read_text())
            out.append((path.name, d.get("measured_on_commit"), d.get("sources")))
        elif path.suffix in (".txt", ".md"):
            text = path.read_text()
            commit = re.search(r"measured on commit ([0-9a-f]{7,40})", text)
            sources = re.search(r"^sources: (.+)$", text, re.M)
            out.append((path.name, commit.group(1) if commit else None, sources.group(1).split() if sources else None))
    return out


@pytest.mark.parametrize("name,commit,sources", _entries(), ids=[e[0] for e in _entries()])
def test_profile_is_of_the_shipped_kernels(name, commit, sources):
    if not (ROOT / ".git").exists() or _git("rev-parse", "HEAD").returncode != 0:
        pytest.skip("no git history here")
    if commit is None and sources is None:
        pytest.skip("a summary of measurements that are not tied to kernel sources")
    assert commit and sources, f"profiles/{name} must name the commit it was measured on and the kernel sources it covers"
    assert _git("cat-file", "-e", f"{commit}^{{commit}}").returncode == 0, f"profiles/{name}: unknown commit {commit}"
    for src in sources:
        assert (ROOT / src).is_file(), f"profiles/{name} names a source that does not exist: {src}"
    later = _git("log", "--oneline", f"{commit}..HEAD", "--", *sources).stdout.strip()
    assert later == "", (f"profiles/{name} was measured on {commit}; these later commits changed the kernels it profiles, "
                         f"re-collect it:\n{later}")
