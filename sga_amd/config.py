"""The args singleton the plugins read their ``sga_*`` flags from
(``sga/config/__init__.py:36-51``): the engine seeds it once with
``set_args``; a plugin constructed before that fails loudly."""

_ARGS = None


def set_args(ns):
    global _ARGS
    _ARGS = ns


def get_args():
    if _ARGS is None:
        raise RuntimeError("sga args not set -- expected set_args() to run before a plugin "
                           "is constructed")
    return _ARGS
