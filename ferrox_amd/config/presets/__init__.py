"""Named configurations for running without a model folder: each `<name>.json` beside this file is a
config.json as a model folder would hold it (the layer sizes of a published model of the family; no weights).
Random weights of these shapes serve measurement and smoke runs, as the reference serves synthetic weights
when it is given no model (ferrox-server/src/model.rs:228-243)."""
from __future__ import annotations

import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def names() -> list:
    return sorted(f[:-5] for f in os.listdir(HERE) if f.endswith(".json"))


def load(name: str) -> dict:
    """The raw config.json dict of the preset `name`."""
    path = os.path.join(HERE, name + ".json")
    if not os.path.isfile(path):
        raise ValueError(f"no configuration named '{name}' (known: {', '.join(names())})")
    with open(path) as f:
        return json.load(f)
