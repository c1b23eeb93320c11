"""A small catalog of model shapes for runs with random weights.

The reference's catalog maps "name:tag" to a download (src/catalog.rs:17-82) and
`find` tries the exact "name:tag", then the name alone (first entry of that name)
(:88-103).  Here an entry is a config.json kept as data beside this file
(shapes/<name>-<tag>.json); the lookup rules are the same.
"""
import json
import os

_SHAPES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "shapes")


def entries():
    """[(name, tag)] of every shape, sorted."""
    out = []
    for f in sorted(os.listdir(_SHAPES)):
        if f.endswith(".json"):
            name, _, tag = f[:-5].rpartition("-")
            out.append((name, tag))
    return out


def find(query):
    """The config.json dictionary for "name:tag", or for "name" its first entry; None if
    there is none."""
    if ":" in query:
        name, tag = query.split(":", 1)
        hits = [(n, t) for n, t in entries() if n == name and t == tag]
    else:
        hits = [(n, t) for n, t in entries() if n == query]
    if not hits:
        return None
    with open(os.path.join(_SHAPES, "%s-%s.json" % hits[0]), "r", encoding="utf-8") as f:
        return json.load(f)
