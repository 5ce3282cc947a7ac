"""Run code written against the reference's flat module layout without editing it.

The reference is three top-level modules that import each other by bare name (``import block_linear_config``,
``from triton_functions import ...`` at block_linear.py:8-12, ``from block_linear import BlockInt8Linear`` in user
code).  :func:`install` registers this package's modules under those names in ``sys.modules``; the config module
is the SAME object under both names, so ``block_linear_config.GROUP_SIZE = 64`` is seen by every operator."""
from __future__ import annotations

import sys

_NAMES = ("block_linear_config", "triton_functions", "block_linear")


def install(force: bool = False) -> None:
    """Make ``import block_linear_config``, ``import triton_functions`` and ``import block_linear`` resolve to
    this package's modules.  Refuses to shadow modules of those names that are already imported from
    elsewhere unless `force` is set."""
    from . import block_linear, block_linear_config, triton_functions
    ours = {"block_linear_config": block_linear_config, "triton_functions": triton_functions, "block_linear": block_linear}
    for name in _NAMES:
        have = sys.modules.get(name)
        if have is not None and have is not ours[name] and not force:
            raise RuntimeError(f"a different module named {name!r} is already imported; pass force=True to replace it")
    for name in _NAMES:
        sys.modules[name] = ours[name]


def uninstall() -> None:
    """Remove the aliases registered by :func:`install` (only those that still point at this package)."""
    from . import block_linear, block_linear_config, triton_functions
    ours = {"block_linear_config": block_linear_config, "triton_functions": triton_functions, "block_linear": block_linear}
    for name in _NAMES:
        if sys.modules.get(name) is ours[name]:
            del sys.modules[name]
