"""Registries from a part's kind (the name a model plan uses) to the class that builds it.

Adding a part means writing a class with the interface of ``parts/base.py`` and registering it
under a new kind; plans may then name it layer by layer.
"""

MIXERS, FEED_FORWARDS, NORMS, EMBEDDINGS, READOUTS, BLOCKS = {}, {}, {}, {}, {}, {}
_TABLES = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS, "embedding": EMBEDDINGS,
           "readout": READOUTS, "block": BLOCKS}


def register(role, kind, cls=None, replace=False):
    """``register("mixer", "attention", Cls)`` or as a decorator ``@register("mixer", "attention")``."""
    table = _TABLES[role]

    def put(c):
        if kind in table and table[kind] is not c and not replace:
            raise ValueError(f"{role} kind {kind!r} is already registered")
        table[kind] = c
        return c

    return put if cls is None else put(cls)


def unregister(role, kind):
    _TABLES[role].pop(kind, None)


def lookup(role, kind):
    table = _TABLES[role]
    if kind not in table:
        raise KeyError(f"no {role} of kind {kind!r}; registered: {sorted(table)}")
    return table[kind]
