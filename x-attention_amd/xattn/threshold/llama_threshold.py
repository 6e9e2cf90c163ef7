"""Per-layer, per-head thresholds of the Llama integration: ``llama_fuse_4``,
``llama_fuse_8``, ``llama_fuse_16`` (one ``[layers][heads]`` table per
antidiagonal stride), the names ``FastPrefillConfig()`` reads when it is built
without a threshold (xattn/src/load_llama.py:249-261 of the reference).

The reference ships tables profiled on Llama-3.1-8B-Instruct in its own
``xattn/threshold/llama_threshold.py``; they are parameters of that model and
are not part of this package.  This module finds tables in one of two places:

* a JSON file ``{"llama_fuse_16": [[...], ...], ...}`` named by the environment
  variable ``XATTN_THRESHOLD_TABLES`` or, by default, ``llama_threshold_tables.json``
  beside this file - what ``python -m xattn.threshold.profile_threshold.profile_threshold
  --write-tables <file>`` produces for the model it profiles;
* or the reference's own module copied over this file (plain module-level
  lists of the same names).

A table that cannot be found raises ``ValueError`` naming both options.
"""
import json
import os

_NAMES = ("llama_fuse_4", "llama_fuse_8", "llama_fuse_16")
DEFAULT_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "llama_threshold_tables.json")


def tables_path():
    return os.environ.get("XATTN_THRESHOLD_TABLES", DEFAULT_PATH)


def load_tables(path=None):
    """``{name: [layers][heads] list}`` from the JSON file, or ``{}`` when it does not exist."""
    path = path or tables_path()
    if not os.path.exists(path):
        return {}
    with open(path) as f:
        data = json.load(f)
    out = {}
    for name, table in data.items():
        if name not in _NAMES:
            continue
        if not (isinstance(table, list) and table and all(isinstance(r, list) and len(r) == len(table[0]) for r in table)):
            raise ValueError(f"{path}: {name} must be a rectangular [layers][heads] list")
        out[name] = [[float(x) for x in row] for row in table]
    return out


def write_tables(path, **tables):
    """Adds or replaces tables (``llama_fuse_<stride>=<[layers][heads] list or tensor>``) in a JSON file."""
    data = load_tables(path) if os.path.exists(path) else {}
    for name, table in tables.items():
        if name not in _NAMES:
            raise ValueError(f"unknown table {name!r}: expected one of {_NAMES}")
        data[name] = [[float(x) for x in row] for row in (table.tolist() if hasattr(table, "tolist") else table)]
    with open(path, "w") as f:
        json.dump(data, f)
    return path


def __getattr__(name):
    if name in _NAMES:
        found = load_tables()
        if name in found:
            return found[name]
        raise ValueError(
            f"no threshold table {name}: neither {tables_path()} holds it (write one with the profiler's "
            "--write-tables, or point XATTN_THRESHOLD_TABLES at one) nor has the reference's "
            "xattn/threshold/llama_threshold.py been copied over " + os.path.abspath(__file__) +
            "; or pass threshold=<float or [layers, heads] tensor> to FastPrefillConfig"
        )
    raise AttributeError(name)
