"""Named config.json files shipped with the package (sizes live in the JSON
files under ``presets/``, not in code)."""
import json
from pathlib import Path

_DIR = Path(__file__).resolve().parent / "presets"


def preset_names():
    return sorted(p.stem for p in _DIR.glob("*.json"))


def preset(name):
    path = _DIR / f"{name}.json"
    if not path.exists():
        raise KeyError(f"unknown preset {name!r}; known: {preset_names()}")
    return json.loads(path.read_text())
